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
