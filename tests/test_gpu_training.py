"""End to end on the GPU: a small MLP whose linears run in FP8 (delayed scaling, bf16 master weights re-quantised
after every optimizer step, fp32 master gradients accumulated by the wgrad epilogue) is trained next to an fp32
twin on the same data.  The reference only checks that such a loop leaves gradients behind
(tests/fp8/test_linear.py:66-83); here the loss curve has to follow the fp32 one."""
import pytest
import torch
from torch import nn

pytestmark = pytest.mark.gpu


def test_fp8_mlp_follows_the_fp32_loss_curve():
    from nanotron_amd.fp8 import FP8Linear
    from nanotron_amd.fp8.optim import attach_requantize_hook

    torch.manual_seed(0)
    T, H, I, steps = 512, 256, 512, 60
    teacher = nn.Sequential(nn.Linear(H, I), nn.GELU(), nn.Linear(I, H)).cuda()
    ref = nn.Sequential(nn.Linear(H, I, bias=False), nn.GELU(), nn.Linear(I, H, bias=False)).cuda()
    fp8 = nn.Sequential(FP8Linear(H, I, bias=False, device="cuda", delayed_scaling=True, amax_history_len=8),
                        nn.GELU(),
                        FP8Linear(I, H, bias=False, device="cuda", delayed_scaling=True, amax_history_len=8))
    with torch.no_grad():
        for a, b in zip(ref.parameters(), fp8.parameters()):
            b.as_subclass(torch.Tensor).copy_(a)
    for lin in (fp8[0], fp8[2]):
        lin.requantize_weight()
    opt_ref = torch.optim.AdamW(ref.parameters(), lr=2e-3)
    opt_fp8 = torch.optim.AdamW(fp8.parameters(), lr=2e-3)
    attach_requantize_hook(opt_fp8, fp8)
    losses_ref, losses_fp8 = [], []
    for step in range(steps):
        x = torch.randn(T, H, device="cuda")
        with torch.no_grad():
            y = teacher(x)
        for model, opt, log in ((ref, opt_ref, losses_ref), (fp8, opt_fp8, losses_fp8)):
            opt.zero_grad(set_to_none=True)
            loss = (model(x) - y).pow(2).mean()
            loss.backward()
            opt.step()
            log.append(loss.item())
    head_ref, tail_ref = sum(losses_ref[:5]) / 5, sum(losses_ref[-5:]) / 5
    head_fp8, tail_fp8 = sum(losses_fp8[:5]) / 5, sum(losses_fp8[-5:]) / 5
    assert tail_ref < 0.5 * head_ref, "the fp32 twin itself must learn"
    assert tail_fp8 < 0.5 * head_fp8
    assert abs(tail_fp8 - tail_ref) <= 0.1 * tail_ref + 1e-4, (tail_fp8, tail_ref)
    # the scaling state moved with the tensors: every role has seen its amax, scales are powers of two
    for lin in (fp8[0], fp8[2]):
        for role, st in lin.scaling.items():
            assert st.initialised and float(st.amax_history[0]) > 0.0, role
            s = float(st.scale)
            assert s > 0 and abs(torch.log2(torch.tensor(s)).item() - round(torch.log2(torch.tensor(s)).item())) < 1e-6


def test_fp8_chain_with_fp8_activations_and_fp8_activation_gradients_trains():
    """Three linears chained through fp8 activations (the TODO at src/nanotron/fp8/linear.py:63-64): forward, no
    high-precision activation is written between the layers (each GEMM epilogue emits the next layer's e4m3 operand);
    backward, no high-precision activation gradient either (each dgrad epilogue emits the e5m2 operand of the layer
    below).  The loss has to follow an fp32 twin's."""
    from nanotron_amd.fp8 import DTypes, FP8Linear, FP8Tensor
    from nanotron_amd.fp8.optim import attach_requantize_hook

    torch.manual_seed(1)
    T, H, I, steps = 512, 256, 384, 80
    # a target the chain of linears cannot fit exactly, so that the loss levels off well above the quantisation noise
    teacher = nn.Sequential(nn.Linear(H, I), nn.GELU(), nn.Linear(I, H)).cuda()
    ref = nn.Sequential(nn.Linear(H, I, bias=False), nn.Linear(I, I, bias=False), nn.Linear(I, H, bias=False)).cuda()
    kw = dict(bias=False, device="cuda", delayed_scaling=True, amax_history_len=8)
    fp8 = nn.Sequential(FP8Linear(H, I, out_dtype=DTypes.FP8E4M3, **kw), FP8Linear(I, I, out_dtype=DTypes.FP8E4M3, **kw),
                        FP8Linear(I, H, **kw))
    with torch.no_grad():
        for a, b in zip(ref.parameters(), fp8.parameters()):
            b.as_subclass(torch.Tensor).copy_(a)
    for lin in fp8:
        lin.requantize_weight()
    opt_ref = torch.optim.AdamW(ref.parameters(), lr=1e-3)
    opt_fp8 = torch.optim.AdamW(fp8.parameters(), lr=1e-3)
    attach_requantize_hook(opt_fp8, fp8)
    losses_ref, losses_fp8 = [], []
    for step in range(steps):
        x = torch.randn(T, H, device="cuda")
        with torch.no_grad():
            y = teacher(x)
        opt_ref.zero_grad(set_to_none=True)
        loss = (ref(x) - y).pow(2).mean()
        loss.backward()
        opt_ref.step()
        losses_ref.append(loss.item())
        opt_fp8.zero_grad(set_to_none=True)
        h1 = fp8[0](x)
        h2 = fp8[1](h1)
        assert isinstance(h1, FP8Tensor) and isinstance(h2, FP8Tensor)
        loss = (fp8[2](h2) - y).pow(2).mean()
        loss.backward()
        opt_fp8.step()
        losses_fp8.append(loss.item())
    head_ref, tail_ref = sum(losses_ref[:5]) / 5, sum(losses_ref[-5:]) / 5
    head_fp8, tail_fp8 = sum(losses_fp8[:5]) / 5, sum(losses_fp8[-5:]) / 5
    assert tail_ref < 0.5 * head_ref, "the fp32 twin itself must learn"
    assert tail_fp8 < 0.5 * head_fp8
    assert abs(tail_fp8 - tail_ref) <= 0.1 * tail_ref + 1e-4, (tail_fp8, tail_ref, head_fp8, head_ref)
    # from the moment the producers' output-gradient roles held a scale, every backward of layers 2 and 3 sent its
    # input gradient down as fp8 bytes; layer 1 has no fp8 input
    assert fp8[1].fp8_grad_inputs_sent >= steps - 3 and fp8[2].fp8_grad_inputs_sent >= steps - 3
    assert fp8[0].fp8_grad_inputs_sent == 0
    for lin in fp8:
        assert lin.weight.grad is not None and bool(torch.isfinite(lin.weight.grad).all())
