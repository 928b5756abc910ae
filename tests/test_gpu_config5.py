"""GPU parity of the benchmark's headline workload at its real shapes, through the product path:
FP8Linear -> batched weight re-quantisation -> forward GEMM -> batched dgrad + wgrad GEMMs whose B operands
are read untransposed (src/nanotron/fp8/linear.py:69-112).  Benchmark configuration 5 (Llama-3-8B block linears,
10 delayed-scaling steps) and configurations 3 / 4 (Llama-7B MLP, wgrad accumulated into fp32 master gradients)."""
import sys

import pytest
import torch

from oracle import fp8_oracle as O
from oracle import step_check as C

pytestmark = pytest.mark.gpu


def _say(msg):
    sys.stderr.write(msg + "\n")
    sys.stderr.flush()


def _build(linears, accumulate=False):
    from nanotron_amd.fp8 import DTypes, FP8Linear, FP8Parameter

    mods, ws = [], []
    for i, (name, K, N) in enumerate(linears):
        lin = FP8Linear(K, N, bias=False, device="cuda", out_dtype=torch.bfloat16, delayed_scaling=True,
                        amax_history_len=16, margin=0, accumulate_grad=accumulate)
        w = C.initial_weight(i, K, N)
        lin.weight = FP8Parameter(w.cuda(), DTypes.FP8E4M3)
        lin.keep_quantised_grad = True   # the checker compares the e5m2 bytes of dY too
        mods.append(lin)
        ws.append(w)
    return mods, ws


def test_is_fp8_available_on_this_gpu():
    # src/nanotron/fp8/utils.py:7-13: the device-name test must say yes on the MI355X the kernels are built for
    from nanotron_amd.fp8.utils import is_fp8_available

    assert is_fp8_available() is True


def test_config5_llama3_8b_block_full_size_10_steps():
    from nanotron_amd.fp8.optim import requantize_fp8_weights

    mods, ws = _build(C.LINEARS)
    refs = C.new_reference_state()
    worst = {"fwd": 0.0, "dgrad": 0.0, "wgrad": 0.0}
    for step in range(10):
        for i, lin in enumerate(mods):
            ws[i] = C.perturbed_weight(ws[i], step, i)
            with torch.no_grad():
                lin.weight.as_subclass(torch.Tensor).copy_(ws[i].cuda())
        requantize_fp8_weights(mods)   # one batched library call once every weight role holds a scale
        for i, ((name, K, N), lin) in enumerate(zip(C.LINEARS, mods)):
            x, gy = C.step_inputs(step, i, K, N)
            xg = x.cuda().requires_grad_(True)
            y = lin(xg)
            xq_gpu = y.grad_fn.saved_tensors[0]
            y.backward(gy.cuda())
            assert lin.weight.grad is None   # bf16 master: the fp32 gradient lives in main_grad
            errs = C.check_layer(f"step {step} {name}", lin, refs[i], x, ws[i], gy, y.detach(), xg.grad,
                                 lin.weight.main_grad, xq_gpu, step, i, gq_gpu=lin.quantised_grad_output)
            for k, v in errs.items():
                worst[k] = max(worst[k], v)
        _say(f"config 5 step {step}: ok, worst rel-L2 so far {worst}")
    # every role has seen ten tensors: the history holds ten positive entries, newest first
    for lin in mods:
        for role in C.ROLES:
            h = lin.scaling[role].amax_history.cpu()
            assert bool((h[:10] > 0).all()) and bool((h[10:] == 0).all())


def test_config3_and_4_llama7b_mlp_through_fp8linear():
    """M = 4096, hidden 4096, intermediate 11008: forward with bf16 outputs, dgrad bf16, wgrad added into a
    pre-filled fp32 master-gradient buffer in the GEMM epilogue; two steps, so that the second one runs the fused
    delayed-scaling kernels and accumulates on top of the first."""
    from nanotron_amd.fp8.optim import requantize_fp8_weights

    linears = [("gate", 4096, 11008), ("up", 4096, 11008), ("down", 11008, 4096)]
    mods, ws = _build(linears, accumulate=True)
    refs = C.new_reference_state()[:3]
    base = [O.normal_tensor(99 + i, (N, K), 1.0, torch.float32) for i, (_, K, N) in enumerate(linears)]
    for lin, b in zip(mods, base):
        lin.weight.main_grad = b.cuda()
    for step in range(2):
        requantize_fp8_weights(mods)
        for i, ((name, K, N), lin) in enumerate(zip(linears, mods)):
            x, gy = C.step_inputs(step, i, K, N)
            xg = x.cuda().requires_grad_(True)
            y = lin(xg)
            xq_gpu = y.grad_fn.saved_tensors[0]
            buf = lin.weight.main_grad
            y.backward(gy.cuda())
            assert lin.weight.main_grad.data_ptr() == buf.data_ptr()   # accumulated in place
            C.check_layer(f"step {step} {name}", lin, refs[i], x, ws[i], gy, y.detach(), xg.grad, lin.weight.main_grad,
                          xq_gpu, step, i, dw_base=base[i], gq_gpu=lin.quantised_grad_output)
            base[i] = lin.weight.main_grad.cpu()
        _say(f"configs 3/4 step {step}: ok")


def test_config5_step_replayed_as_a_graph_matches_eager_launches():
    """The benchmark step at its real shapes captured once as a HIP graph (weight re-quantisation, then for every
    linear: quantise X, forward GEMM, quantise dY, dgrad + wgrad launch) and replayed eight times with fresh inputs
    copied into its static buffers, against an eager twin: outputs, gradients, fp8 weight bytes and the whole scaling
    state bit for bit after every replay, with eager work and synchronisations between the replays."""
    from nanotron_amd.fp8.optim import requantize_fp8_weights

    g_mods, ws = _build(C.LINEARS)
    e_mods, _ = _build(C.LINEARS)
    sx = [torch.zeros(C.TOKENS, K, dtype=torch.bfloat16, device="cuda", requires_grad=True) for _, K, _ in C.LINEARS]
    sgy = [torch.zeros(C.TOKENS, N, dtype=torch.bfloat16, device="cuda") for _, _, N in C.LINEARS]

    def load(step):
        """This step's weights into both sets of modules, its inputs into the static buffers; returns the inputs."""
        ins = []
        for i, (name, K, N) in enumerate(C.LINEARS):
            ws[i] = C.perturbed_weight(ws[i], step, i)
            w = ws[i].cuda()
            x, gy = C.step_inputs(step, i, K, N)
            x, gy = x.cuda(), gy.cuda()
            with torch.no_grad():
                g_mods[i].weight.as_subclass(torch.Tensor).copy_(w)
                e_mods[i].weight.as_subclass(torch.Tensor).copy_(w)
                sx[i].copy_(x)
                sgy[i].copy_(gy)
            ins.append((x, gy))
        return ins

    def run(mods, xs, gys):
        requantize_fp8_weights(mods)
        ys = []
        for lin, x, gy in zip(mods, xs, gys):
            x.grad = None
            y = lin(x)
            y.backward(gy)
            ys.append(y)
        return ys

    side = torch.cuda.Stream()
    for step in range(2):   # every role gets its first scale (a role's first quantisation reads its amax on the host)
        ins = load(step)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            run(g_mods, sx, sgy)
        torch.cuda.current_stream().wait_stream(side)
        run(e_mods, [x.requires_grad_(True) for x, _ in ins], [gy for _, gy in ins])
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_ys = run(g_mods, sx, sgy)
    for step in range(2, 10):
        ins = load(step)
        graph.replay()
        xe = [x.requires_grad_(True) for x, _ in ins]
        e_ys = run(e_mods, xe, [gy for _, gy in ins])
        _ = float((e_ys[1][:64].float() @ e_ys[1][:64].float().t()).sum())   # unrelated eager work and a synchronisation
        for i, (name, _, _) in enumerate(C.LINEARS):
            tag = f"step {step} {name}"
            assert torch.equal(g_ys[i], e_ys[i]), f"{tag}: Y of the replay differs"
            assert torch.equal(sx[i].grad, xe[i].grad), f"{tag}: dX of the replay differs"
            assert torch.equal(g_mods[i].weight.main_grad, e_mods[i].weight.main_grad), f"{tag}: dW of the replay differs"
            assert torch.equal(g_mods[i].weight.data.as_subclass(torch.Tensor),
                               e_mods[i].weight.data.as_subclass(torch.Tensor)), f"{tag}: fp8 weight bytes differ"
            for role in C.ROLES:
                assert torch.equal(g_mods[i].scaling[role]._buf, e_mods[i].scaling[role]._buf), f"{tag} {role}: scaling state differs"
        _say(f"config 5 graph replay, step {step}: identical to the eager launches")
