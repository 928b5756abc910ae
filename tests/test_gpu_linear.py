"""GPU tests of FP8Linear: the reference's own test cases (tests/fp8/test_linear.py) re-stated
against this package, then the same checks tightened with the oracle on non-square shapes, real
upstream gradients and delayed scaling over several steps."""
import pytest
import torch
from torch import nn
from torch.optim import Adam

from oracle import fp8_oracle as O

pytestmark = pytest.mark.gpu

REL_L2 = 1e-3


# ------------------------------------------------------------------ reference tests, mirrored
@pytest.mark.parametrize("is_bias", [True, False])
def test_fp8_linear_forward_pass(is_bias):
    # tests/fp8/test_linear.py:8-25
    from nanotron_amd.fp8 import DTypes, FP8Linear, FP8Parameter

    input = torch.randn(16, 16, device="cuda", dtype=torch.float32)
    ref_input = input.detach().clone()
    ref_linear = nn.Linear(16, 16, bias=is_bias, device="cuda", dtype=torch.float32)
    fp8_linear = FP8Linear(16, 16, bias=is_bias, device="cuda:0")
    fp8_linear.weight = FP8Parameter(ref_linear.weight.detach().clone(), DTypes.FP8E4M3)
    if is_bias:
        fp8_linear.bias.data = ref_linear.bias.detach().clone()
    ref_output = ref_linear(ref_input)
    output = fp8_linear(input)
    assert isinstance(output, torch.Tensor)
    assert output.dtype == torch.float32
    assert torch.allclose(output, ref_output, rtol=0, atol=0.1)


@pytest.mark.parametrize("input_requires_grad", [True, False])
@pytest.mark.parametrize("device", ["cuda:0", "cpu"])
def test_fp8_linear_backward_pass(input_requires_grad, device):
    # tests/fp8/test_linear.py:29-49 (plus the input-gradient check the reference left disabled)
    from nanotron_amd.fp8 import DTypes, FP8Linear, FP8Tensor

    input = torch.randn(16, 16, device=device, dtype=torch.float32, requires_grad=input_requires_grad)
    ref_input = input.detach().clone().requires_grad_(True)
    ref_linear = nn.Linear(16, 16, device=device, dtype=torch.float32)
    fp8_linear = FP8Linear(16, 16, device=device)
    if device == "cpu":
        fp8_linear.weight.data = ref_linear.weight.detach().clone()
    else:
        fp8_linear.weight.data = FP8Tensor(ref_linear.weight.detach().clone(), dtype=DTypes.FP8E4M3)
    fp8_linear.bias.data = ref_linear.bias.detach().clone()
    ref_linear(ref_input).sum().backward()
    fp8_linear(input).sum().backward()
    assert torch.allclose(fp8_linear.bias.grad, ref_linear.bias.grad, 0, 0.1)
    if device == "cpu":
        assert torch.allclose(fp8_linear.weight.grad, ref_linear.weight.grad, 0.1, 0.1)
        return
    # Against the un-quantised fp32 layer the reference asserts rtol=atol=0.1.  Each e4m3 input carries
    # up to 2^-4 relative rounding error and dW sums 16 of them, so that bound is itself noisy (the
    # reference never runs this test in CI); here it is asserted against the oracle, which computes
    # the same quantised arithmetic, and only loosely against the fp32 layer.
    xq = O.quantise_current(ref_input.detach().cpu(), O.E4M3)
    wq = O.quantise_current(ref_linear.weight.detach().cpu(), O.E4M3)
    gq = O.quantise_current(torch.ones(16, 16), O.E5M2)
    assert torch.allclose(fp8_linear.weight.grad.cpu(), O.linear_wgrad(gq, xq), 1e-3, 1e-3)
    assert torch.allclose(fp8_linear.weight.grad, ref_linear.weight.grad, 0.1, 0.5)
    if input_requires_grad:
        assert torch.allclose(input.grad.cpu(), O.linear_dgrad(gq, wq), 1e-3, 1e-3)
        assert torch.allclose(input.grad, ref_input.grad, 0.1, 0.1)


def test_fp8_linear_attrs():
    # tests/fp8/test_linear.py:55-59
    from nanotron_amd.fp8 import FP8Linear

    fp8_linear = FP8Linear(16, 16, device="cuda:0")
    assert next(fp8_linear.parameters()) is not None
    assert all(p.requires_grad for p in fp8_linear.parameters()) is True
    assert set(fp8_linear.fp8_meta) == {"input_grad", "weight_grad", "output_grad"}
    assert fp8_linear.fp8_meta["input_grad"].scale.item() == 256.0
    assert fp8_linear.fp8_meta["output_grad"].scale.item() == 32768.0


def test_fp8_model_bwd():
    # tests/fp8/test_linear.py:66-83
    from nanotron_amd.fp8 import FP8Linear

    H, L, E = 128, 5, 3
    input = torch.randn(H, H, device="cuda", requires_grad=True)
    model = nn.Sequential(*[nn.Sequential(FP8Linear(H, H, device="cuda"), nn.ReLU()) for _ in range(L)])
    optim = Adam(model.parameters(), lr=1e-3)
    for _ in range(E):
        optim.zero_grad()
        model(input).sum().backward()
        optim.step()
    assert all(p.grad is not None for p in model.parameters())


# ------------------------------------------------------------------ oracle-tight checks
def _oracle_step(x, w, gy, sx=None, sw=None, sg=None):
    xq = sx.quantise(x) if sx else O.quantise_current(x, O.E4M3)
    wq = sw.quantise(w) if sw else O.quantise_current(w, O.E4M3)
    gq = sg.quantise(gy) if sg else O.quantise_current(gy, O.E5M2)
    return xq, wq, gq, O.linear_forward(xq, wq), O.linear_dgrad(gq, wq), O.linear_wgrad(gq, xq)


@pytest.mark.parametrize("shape", [(48, 32, 80), (256, 384, 128), (100, 36, 52), (2048, 1024, 1024)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_fwd_bwd_nonsquare_real_gradients(shape, dtype):
    from nanotron_amd.fp8 import DTypes, FP8Linear, FP8Parameter

    M, K, N = shape
    x = O.normal_tensor(1, (M, K), 1.0, dtype)
    w = O.normal_tensor(2, (N, K), 0.02, torch.float32)
    gy = O.normal_tensor(3, (M, N), 1e-3, torch.float32)
    lin = FP8Linear(K, N, bias=False, device="cuda")
    lin.weight = FP8Parameter(w.cuda(), DTypes.FP8E4M3)
    xg = x.cuda().requires_grad_(True)
    y = lin(xg)
    assert y.dtype == torch.float32 and y.shape == (M, N)
    y.backward(gy.cuda())
    xq, wq, gq, y_ref, dx_ref, dw_ref = _oracle_step(x, w, gy)
    assert torch.equal(lin.weight.data.cpu().as_subclass(torch.Tensor), wq.q)
    assert O.rel_l2(y.detach().cpu(), y_ref) <= REL_L2
    assert xg.grad.dtype == dtype
    assert O.rel_l2(xg.grad.float().cpu(), dx_ref.to(dtype).float()) <= (REL_L2 if dtype == torch.float32 else 4e-3)
    assert lin.weight.grad.dtype == torch.float32 and lin.weight.grad.shape == (N, K)
    assert O.rel_l2(lin.weight.grad.cpu(), dw_ref) <= REL_L2


def test_fp8matmul_apply_with_the_references_four_arguments():
    """`_FP8Matmul.apply(input, weight, fp8_meta, phony)` exactly as src/nanotron/fp8/linear.py:60 calls it (no module,
    no bias, no handle): current scaling, fp32 output; forward, dX and the `weight.grad` side effect against the oracle."""
    from nanotron_amd.fp8 import DTypes, FP8Linear, FP8Parameter
    from nanotron_amd.fp8.linear import _FP8Matmul

    M, K, N = 192, 160, 272
    x = O.normal_tensor(41, (M, K), 1.0, torch.float32)
    w = O.normal_tensor(42, (N, K), 0.02, torch.float32)
    gy = O.normal_tensor(43, (M, N), 1e-3, torch.float32)
    lin = FP8Linear(K, N, bias=False, device="cuda")   # only for its fp8_meta dictionary, as linear.py:33-49 builds it
    weight = FP8Parameter(w.cuda(), DTypes.FP8E4M3)
    xg = x.cuda().requires_grad_(True)
    phony = torch.empty(0, device="cuda", requires_grad=True)
    output, _ = _FP8Matmul.apply(xg, weight, lin.fp8_meta, phony)
    assert output.dtype == torch.float32 and output.shape == (M, N)
    output.backward(gy.cuda())
    xq, wq, gq, y_ref, dx_ref, dw_ref = _oracle_step(x, w, gy)
    assert O.rel_l2(output.detach().cpu(), y_ref) <= REL_L2
    assert O.rel_l2(xg.grad.cpu(), dx_ref) <= REL_L2
    assert weight.grad.dtype == torch.float32 and O.rel_l2(weight.grad.cpu(), dw_ref) <= REL_L2
    assert phony.grad is None


def test_linear_3d_input_bias_and_out_dtype():
    from nanotron_amd.fp8 import DTypes, FP8Linear, FP8Parameter

    B, S, K, N = 2, 24, 64, 48
    x = O.normal_tensor(4, (B, S, K), 1.0, torch.bfloat16)
    w = O.normal_tensor(5, (N, K), 0.05, torch.float32)
    b = O.normal_tensor(6, (N,), 0.1, torch.float32)
    lin = FP8Linear(K, N, bias=True, device="cuda", out_dtype=torch.bfloat16)
    lin.weight = FP8Parameter(w.cuda(), DTypes.FP8E4M3)
    lin.bias.data = b.cuda()
    xg = x.cuda().requires_grad_(True)
    y = lin(xg)
    assert y.shape == (B, S, N)
    y.float().sum().backward()
    xq = O.quantise_current(x.reshape(-1, K), O.E4M3)
    wq = O.quantise_current(w, O.E4M3)
    y_ref = O.linear_forward(xq, wq, torch.bfloat16).reshape(B, S, N) + b
    assert O.rel_l2(y.detach().float().cpu(), y_ref.float()) <= 8e-3
    assert xg.grad.shape == (B, S, K) and lin.bias.grad.shape == (N,)
    assert torch.allclose(lin.bias.grad.cpu(), torch.full((N,), float(B * S)))


def test_accumulate_grad_into_fp32_master_buffer():
    # optim/gradient_accumulator.py:222 `fp32_grad.add_(grad)` folded into the wgrad epilogue
    from nanotron_amd.fp8 import DTypes, FP8Linear, FP8Parameter

    M, K, N = 192, 128, 160
    w = O.normal_tensor(12, (N, K), 0.02, torch.float32)
    lin = FP8Linear(K, N, bias=False, device="cuda", accumulate_grad=True)
    lin.weight = FP8Parameter(w.cuda(), DTypes.FP8E4M3)
    total = torch.zeros(N, K)
    for step in range(3):
        x = O.normal_tensor(20 + step, (M, K), 1.0, torch.bfloat16)
        gy = O.normal_tensor(30 + step, (M, N), 1e-3, torch.bfloat16)
        lin(x.cuda().requires_grad_(True)).backward(gy.cuda().float())
        *_, dw_ref = _oracle_step(x, w, gy.float())
        total = total + dw_ref
        assert O.rel_l2(lin.weight.grad.cpu(), total) <= REL_L2


def test_bf16_master_weight_keeps_fp32_gradient_as_main_grad():
    # bf16 parameters cannot carry an fp32 `.grad`: the fp32 wgrad result goes to `.main_grad`
    from nanotron_amd.fp8 import DTypes, FP8Linear, FP8Parameter

    M, K, N = 320, 256, 384
    w = O.normal_tensor(41, (N, K), 0.02, torch.bfloat16)
    for accumulate in (False, True):
        lin = FP8Linear(K, N, bias=False, device="cuda", out_dtype=torch.bfloat16, accumulate_grad=accumulate)
        lin.weight = FP8Parameter(w.cuda(), DTypes.FP8E4M3)
        assert lin.weight.dtype == torch.bfloat16
        total = torch.zeros(N, K)
        for step in range(2):
            x = O.normal_tensor(50 + step, (M, K), 1.0, torch.bfloat16)
            gy = O.normal_tensor(60 + step, (M, N), 1e-3, torch.bfloat16)
            xg = x.cuda().requires_grad_(True)
            lin.requantize_weight()
            lin(xg).backward(gy.cuda())
            *_, dx_ref, dw_ref = _oracle_step(x, w, gy)
            total = total + dw_ref if accumulate else dw_ref
            assert lin.weight.grad is None
            assert lin.weight.main_grad.dtype == torch.float32
            assert O.rel_l2(lin.weight.main_grad.cpu(), total) <= REL_L2
            assert O.rel_l2(xg.grad.float().cpu(), dx_ref) <= 4e-3  # bf16 input gradient


def test_delayed_scaling_ten_steps_llama_like_block_reduced():
    """Benchmark config 5 in miniature (same structure: 5 linears, fwd+bwd, 10 steps, history 16,
    weights perturbed every step), every amax / scale / history compared bit-exact per step."""
    from nanotron_amd.fp8 import FP8Linear

    M = 256
    shapes = {"qkv": (512, 768), "o": (512, 512), "gate": (512, 1792), "up": (512, 1792), "down": (1792, 512)}
    lins, refs, ws = {}, {}, {}
    for i, (name, (K, N)) in enumerate(shapes.items()):
        lins[name] = FP8Linear(K, N, bias=False, device="cuda", delayed_scaling=True, out_dtype=torch.bfloat16)
        ws[name] = O.normal_tensor(500 + i, (N, K), 0.02, torch.float32)
        refs[name] = {r: O.DelayedScaling(O.E4M3 if r != "output_grad" else O.E5M2) for r in ("input", "weight", "output_grad")}
    for step in range(10):
        for i, (name, (K, N)) in enumerate(shapes.items()):
            lin, ref = lins[name], refs[name]
            ws[name] = ws[name] + O.normal_tensor(9000 + 10 * step + i, (N, K), 0.002 * (1 + step % 3), torch.float32)
            with torch.no_grad():
                lin.weight.as_subclass(torch.Tensor).copy_(ws[name].cuda())
            lin.requantize_weight()
            x = O.normal_tensor(7000 + 10 * step + i, (M, K), 1.0 + 0.3 * (step % 4), torch.bfloat16)
            gy = O.normal_tensor(8000 + 10 * step + i, (M, N), 1e-3 * (1 + step % 2), torch.bfloat16)
            xg = x.cuda().requires_grad_(True)
            y = lin(xg)
            y.backward(gy.cuda())
            xq, wq, gq, y_ref, dx_ref, dw_ref = _oracle_step(x, ws[name], gy, ref["input"], ref["weight"], ref["output_grad"])
            for role in ("input", "weight", "output_grad"):
                st, rf = lin.scaling[role], ref[role]
                assert st.scale.item() == rf.scale.item(), (step, name, role)
                assert torch.equal(st.amax_history.cpu(), rf.hist), (step, name, role)
            assert torch.equal(lin.weight.data.cpu().as_subclass(torch.Tensor), wq.q), (step, name)
            assert lin.weight.data.fp8_meta.scale.item() == wq.scale.item()
            assert O.rel_l2(y.detach().float().cpu(), y_ref) <= 4e-3, (step, name)
            assert O.rel_l2(xg.grad.float().cpu(), dx_ref) <= 4e-3, (step, name)
            assert O.rel_l2(lin.weight.grad.cpu(), dw_ref) <= REL_L2, (step, name)
