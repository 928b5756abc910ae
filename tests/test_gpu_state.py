"""GPU tests of the callers either side of the path: FP8 state in checkpoints (a resumed run continues
the delayed-scaling trajectory bit for bit) and weight re-quantisation after an optimizer step."""
import io

import pytest
import torch
from torch import nn

from oracle import fp8_oracle as O

pytestmark = pytest.mark.gpu


def _block(delayed):
    from nanotron_amd.fp8 import FP8Linear

    torch.manual_seed(7)
    return nn.Sequential(
        FP8Linear(256, 384, bias=True, device="cuda", delayed_scaling=delayed, out_dtype=torch.bfloat16),
        FP8Linear(384, 256, bias=False, device="cuda", delayed_scaling=delayed, out_dtype=torch.bfloat16),
    )


def _step(model, i, lr=1e-2):
    """One training step with plain SGD on the master weights; returns everything a resume must reproduce."""
    from nanotron_amd.fp8.optim import requantize_fp8_weights

    x = O.normal_tensor(100 + i, (320, 256), 1.0 + 0.2 * (i % 3), torch.bfloat16).cuda().requires_grad_(True)
    gy = O.normal_tensor(200 + i, (320, 256), 1e-3, torch.bfloat16).cuda()
    for lin in model:
        lin.weight.grad = None
    y = model(x)
    y.backward(gy)
    with torch.no_grad():
        for lin in model:
            lin.weight.as_subclass(torch.Tensor).add_(lin.weight.grad, alpha=-lr)
    requantize_fp8_weights(model)
    out = [y.detach().clone(), x.grad.clone()]
    for lin in model:
        out += [lin.weight.grad.clone(), lin.weight.data.as_subclass(torch.Tensor).clone(),
                lin.weight.data.transposed().as_subclass(torch.Tensor).clone(), lin.weight.fp8_meta.scale.clone()]
        if lin.scaling is not None:
            out += [st._buf.clone() for st in lin.scaling.values()]
    return out


@pytest.mark.parametrize("delayed", [True, False])
def test_checkpoint_resume_is_bit_exact(delayed):
    a = _block(delayed)
    for i in range(3):
        _step(a, i)
    buf = io.BytesIO()
    torch.save(a.state_dict(), buf)
    want = [_step(a, i) for i in range(3, 6)]

    b = _block(delayed)
    for lin in b:  # a fresh model with different weights and histories
        with torch.no_grad():
            lin.weight.as_subclass(torch.Tensor).mul_(1.5)
    buf.seek(0)
    sd = torch.load(buf, weights_only=True)
    keys = [k for k in sd if "fp8_state." in k]
    assert (len(keys) == 8) if delayed else (len(keys) == 0)
    assert all(isinstance(sd[k], torch.Tensor) and sd[k].dtype == torch.float32 for k in keys)
    res = b.load_state_dict(sd, strict=True)
    assert not res.missing_keys and not res.unexpected_keys
    got = [_step(b, i) for i in range(3, 6)]
    for ws, gs in zip(want, got):
        assert len(ws) == len(gs)
        for w, g in zip(ws, gs):
            assert torch.equal(w, g)


def test_state_dict_without_fp8_state_still_loads():
    # a checkpoint written by a plain nn.Linear (or by the reference's FP8Linear) carries weight / bias only
    from nanotron_amd.fp8 import FP8Linear

    ref = nn.Linear(128, 192, device="cuda")
    lin = FP8Linear(128, 192, device="cuda")
    res = lin.load_state_dict(ref.state_dict(), strict=True)
    assert not res.missing_keys and not res.unexpected_keys
    wq = O.quantise_current(ref.weight.detach().cpu(), O.E4M3)
    assert torch.equal(lin.weight.data.cpu().as_subclass(torch.Tensor), wq.q)
    assert torch.equal(lin.weight.data.transposed().cpu().as_subclass(torch.Tensor), wq.q.t().contiguous())
    # with delayed scaling the state keys are required by a strict load and optional otherwise
    lin2 = FP8Linear(128, 192, device="cuda", delayed_scaling=True)
    with pytest.raises(RuntimeError):
        lin2.load_state_dict(ref.state_dict(), strict=True)
    res = lin2.load_state_dict(ref.state_dict(), strict=False)
    assert all("fp8_state." in k for k in res.missing_keys) and len(res.missing_keys) == 3


def test_optimizer_hook_requantises_after_every_step():
    from nanotron_amd.fp8 import FP8Linear
    from nanotron_amd.fp8.optim import attach_requantize_hook

    torch.manual_seed(3)
    model = nn.Sequential(FP8Linear(128, 128, device="cuda"), nn.ReLU(), FP8Linear(128, 64, device="cuda"))
    opt = torch.optim.SGD(model.parameters(), lr=0.5)
    handle = attach_requantize_hook(opt, model)
    x = torch.randn(64, 128, device="cuda")
    for _ in range(2):
        opt.zero_grad()
        model(x).sum().backward()
        before = [m.weight.data.as_subclass(torch.Tensor).clone() for m in model if isinstance(m, FP8Linear)]
        opt.step()
        lins = [m for m in model if isinstance(m, FP8Linear)]
        for lin, old in zip(lins, before):
            wq = O.quantise_current(lin.weight.as_subclass(torch.Tensor).detach().cpu(), O.E4M3)
            assert torch.equal(lin.weight.data.cpu().as_subclass(torch.Tensor), wq.q)
            assert torch.equal(lin.weight.data.transposed().cpu().as_subclass(torch.Tensor), wq.q.t().contiguous())
            assert float(lin.weight.fp8_meta.scale) == float(wq.scale)
            assert not torch.equal(lin.weight.data.as_subclass(torch.Tensor), old)
    handle.remove()
    opt.zero_grad()
    model(x).sum().backward()
    before = model[0].weight.data.as_subclass(torch.Tensor).clone()
    opt.step()
    assert torch.equal(model[0].weight.data.as_subclass(torch.Tensor), before)  # detached: no refresh any more


def test_step_replayed_as_a_graph_matches_eager():
    """The library allocates nothing, synchronises nothing and leaves its reduction workspace zero, so a
    training step can be captured once and replayed: three replays with fresh inputs, with eager work and
    synchronisations in between, against an eager twin that starts from the same state."""
    import copy

    from nanotron_amd.fp8 import FP8Linear
    from nanotron_amd.fp8.optim import requantize_fp8_weights

    def build():
        torch.manual_seed(11)
        return nn.Sequential(FP8Linear(256, 512, bias=False, device="cuda", delayed_scaling=True, out_dtype=torch.bfloat16),
                             FP8Linear(512, 256, bias=False, device="cuda", delayed_scaling=True, out_dtype=torch.bfloat16))

    def inputs(i):
        return (O.normal_tensor(300 + i, (384, 256), 1.0 + 0.1 * i, torch.bfloat16).cuda(),
                O.normal_tensor(400 + i, (384, 256), 1e-3, torch.bfloat16).cuda())

    def step(model, x, gy):
        requantize_fp8_weights(model)
        x.grad = None
        y = model(x)
        y.backward(gy)
        return y

    g_model, e_model = build(), build()
    sx = torch.zeros(384, 256, dtype=torch.bfloat16, device="cuda", requires_grad=True)
    sgy = torch.zeros(384, 256, dtype=torch.bfloat16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):   # warm-up on the capture stream: every scaling state has seen an amax
        for i in range(2):
            x, gy = inputs(i)
            with torch.no_grad():
                sx.copy_(x)
                sgy.copy_(gy)
            step(g_model, sx, sgy)
    torch.cuda.current_stream().wait_stream(side)
    for i in range(2):
        x, gy = inputs(i)
        step(e_model, x.requires_grad_(True), gy)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    x, gy = inputs(2)
    with torch.no_grad():
        sx.copy_(x)
        sgy.copy_(gy)
    with torch.cuda.graph(graph):
        sy = step(g_model, sx, sgy)
    # capture does not execute: bring the eager twin to the same point by not stepping it either
    for i in range(2, 5):
        x, gy = inputs(i)
        with torch.no_grad():
            sx.copy_(x)
            sgy.copy_(gy)
        graph.replay()
        xe = x.clone().requires_grad_(True)
        ye = step(e_model, xe, gy)
        _ = (ye.float() @ ye.float().t()).sum().item()   # unrelated eager work and a synchronisation in between
        assert torch.equal(sy, ye)
        assert torch.equal(sx.grad, xe.grad)
        for lg, le in zip(g_model, e_model):
            assert torch.equal(lg.weight.main_grad if lg.weight.dtype != torch.float32 else lg.weight.grad,
                               le.weight.main_grad if le.weight.dtype != torch.float32 else le.weight.grad)
            for role in lg.scaling:
                assert torch.equal(lg.scaling[role]._buf, le.scaling[role]._buf)


def test_a_fresh_layers_first_steps_replay_as_a_graph():
    """No quantisation reads anything back to the host, not even a role's first (which scales from the tensor's own
    amax and is told apart from the later ones by a flag in device memory): a step captured on layers that have never
    run replays as their first, second and third step, bit for bit like an eager twin's."""
    from nanotron_amd.fp8 import FP8Linear
    from nanotron_amd.fp8.optim import requantize_fp8_weights

    def build():
        torch.manual_seed(23)
        return nn.Sequential(FP8Linear(256, 384, bias=False, device="cuda", delayed_scaling=True, out_dtype=torch.bfloat16),
                             FP8Linear(384, 256, bias=False, device="cuda", delayed_scaling=True, out_dtype=torch.bfloat16))

    def step(model, x, gy):
        requantize_fp8_weights(model)
        x.grad = None
        y = model(x)
        y.backward(gy)
        return y

    g_model, e_model = build(), build()
    sx = torch.zeros(320, 256, dtype=torch.bfloat16, device="cuda", requires_grad=True)
    sgy = torch.zeros(320, 256, dtype=torch.bfloat16, device="cuda")
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        sy = step(g_model, sx, sgy)
    for i in range(3):
        x = O.normal_tensor(500 + i, (320, 256), 1.0 + i, torch.bfloat16).cuda()
        gy = O.normal_tensor(600 + i, (320, 256), 1e-3, torch.bfloat16).cuda()
        with torch.no_grad():
            sx.copy_(x)
            sgy.copy_(gy)
        graph.replay()
        xe = x.clone().requires_grad_(True)
        ye = step(e_model, xe, gy)
        torch.cuda.synchronize()
        assert torch.equal(sy, ye), i
        assert torch.equal(sx.grad, xe.grad), i
        for lg, le in zip(g_model, e_model):
            assert torch.equal(lg.weight.grad, le.weight.grad), i
            for role in lg.scaling:
                assert torch.equal(lg.scaling[role]._buf, le.scaling[role]._buf), (i, role)
                assert torch.equal(lg.scaling[role]._flag, le.scaling[role]._flag), (i, role)
    assert all(st.initialised for lg in g_model for st in lg.scaling.values())
