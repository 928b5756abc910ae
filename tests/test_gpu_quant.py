"""GPU parity: amax / scale / history / fp8 bytes of the HIP kernels against the CPU oracle,
bit for bit, through the C ABI (nanotron_amd._native) and through the FP8Tensor API."""
import math

import numpy as np
import pytest
import torch

from oracle import fp8_oracle as O

pytestmark = pytest.mark.gpu

FMTS = [O.E4M3, O.E5M2]


def _api():
    from nanotron_amd import _native as nt
    from nanotron_amd.fp8 import DTypes, DelayedScaling, FP8Tensor
    from nanotron_amd.fp8 import tensor as T

    return nt, DTypes, DelayedScaling, FP8Tensor, T


def _dt(fmt):
    from nanotron_amd.fp8 import DTypes

    return DTypes.FP8E4M3 if fmt == O.E4M3 else DTypes.FP8E5M2


def _cast(x_gpu, scale, fmt):
    """C ABI: ntfp8_cast_to_fp8 with an explicit scale."""
    nt, *_ = _api()
    x = x_gpu.contiguous()
    s = torch.tensor(scale, dtype=torch.float32, device="cuda")
    out = torch.empty(x.shape, dtype=torch.uint8, device="cuda")
    cols = x.shape[-1] if x.dim() >= 2 else x.numel()
    nt.check(nt.lib.ntfp8_cast_to_fp8(x.data_ptr(), nt.TORCH_TO_NT[x.dtype], x.numel() // cols, cols, s.data_ptr(),
                                      nt.E4M3 if fmt == O.E4M3 else nt.E5M2, out.data_ptr(), None,
                                      nt.stream_ptr(x.device)), "cast")
    return out.cpu()


def same_float(a: float, b: float) -> bool:
    return (math.isnan(a) and math.isnan(b)) or a == b


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("src", [torch.bfloat16, torch.float16])
def test_cast_exhaustive_16bit_patterns(fmt, src):
    bits = torch.arange(0, 0x10000, dtype=torch.int32).to(torch.int16)
    x = bits.view(src)
    xg = x.cuda()
    for k in list(range(-3, 16)) + [-20, 40, 100]:
        s = 2.0 ** k
        want = O.cast_to_fp8(x, torch.tensor(s, dtype=torch.float32), fmt)
        got = _cast(xg, s, fmt)
        bad = (want != got).nonzero().flatten()
        assert bad.numel() == 0, (f"scale 2^{k}: {bad.numel()} mismatches, first pattern "
                                  f"{int(bits[bad[0]]) & 0xffff:#06x} want {int(want[bad[0]]):#04x} got {int(got[bad[0]]):#04x}")


@pytest.mark.parametrize("fmt", FMTS)
def test_cast_fp32_midpoints_random_and_nonpow2_scales(fmt):
    tab = O.decode_table(fmt)
    maxc = 0x7E if fmt == O.E4M3 else 0x7B
    mags = tab[: maxc + 1]
    mids = ((mags[:-1] + mags[1:]) / 2).astype(np.float32)
    pts = np.concatenate([mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(np.inf)),
                          mags.astype(np.float32)])
    pts = np.concatenate([pts, -pts])
    x = torch.from_numpy(pts)
    assert torch.equal(_cast(x.cuda(), 1.0, fmt), O.cast_to_fp8(x, torch.tensor(1.0), fmt))
    g = torch.Generator().manual_seed(11)
    x = torch.randn(1 << 20, generator=g) * torch.exp(torch.randn(1 << 20, generator=g) * 4)
    x[::1001] = float("nan")
    x[1::1001] = float("inf")
    x[2::1001] = -float("inf")
    x[3::1001] = -0.0
    neg_nan = torch.tensor([-4194304], dtype=torch.int32).view(torch.float32)  # 0xffc00000
    x[4::1001] = neg_nan
    for s in (0.37, 1.0, 256.0, 3.1e4, 2.0 ** -30):
        sf = float(np.float32(s))
        want = O.cast_to_fp8(x, torch.tensor(sf, dtype=torch.float32), fmt)
        assert torch.equal(_cast(x.cuda(), sf, fmt), want), f"scale {s}"


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(4, 4), (64, 64), (1, 1), (7,), (3, 5, 17), (128, 128), (256, 384), (1000, 33)])
def test_fp8tensor_current_scaling_bit_exact(fmt, dtype, shape):
    nt, DTypes, _, FP8Tensor, T = _api()
    seed = sum(shape) * 7 + len(shape) + {torch.float32: 0, torch.bfloat16: 1000, torch.float16: 2000}[dtype]
    x = O.normal_tensor(seed, shape, 1.7, dtype)
    x.view(-1)[0] = -0.0  # quantises to the code 0x80, which must come back as -0 in every output dtype
    want = O.quantise_current(x, fmt)
    got = FP8Tensor(x.cuda(), _dt(fmt))
    assert got.dtype == torch.uint8 and got.shape == x.shape and want.q.view(-1)[0] == 0x80
    assert got.fp8_meta.amax.item() == want.amax.item()
    assert got.fp8_meta.scale.item() == want.scale.item()
    assert torch.equal(got.cpu().as_subclass(torch.Tensor), want.q)
    # dequantise through the C ABI against the oracle, every output dtype
    for od in (torch.float32, torch.bfloat16, torch.float16):
        back = T.convert_tensor_from_fp8(got, got.fp8_meta, od).cpu()
        ref = O.cast_from_fp8(want.q, want.scale, fmt, od)
        assert back.dtype == od and torch.equal(back.view(torch.int16 if od != torch.float32 else torch.int32),
                                                ref.view(torch.int16 if od != torch.float32 else torch.int32))


@pytest.mark.parametrize("fmt", FMTS)
def test_misaligned_views_and_noncontiguous_inputs(fmt):
    _, _, _, FP8Tensor, _ = _api()
    base = O.normal_tensor(5, (4099,), 1.0, torch.bfloat16)
    bg = base.cuda()
    for off in (1, 3, 8):
        want = O.quantise_current(base[off:], fmt)
        got = FP8Tensor(bg[off:], _dt(fmt))
        assert torch.equal(got.cpu().as_subclass(torch.Tensor), want.q) and got.fp8_meta.amax.item() == want.amax.item()
    m = O.normal_tensor(6, (130, 70), 1.0, torch.float32)
    want = O.quantise_current(m.t(), fmt)
    got = FP8Tensor(m.cuda().t(), _dt(fmt))
    assert got.shape == (70, 130) and torch.equal(got.cpu().as_subclass(torch.Tensor), want.q)


@pytest.mark.parametrize("fmt", FMTS)
def test_special_values_nan_inf_zero(fmt):
    _, _, _, FP8Tensor, _ = _api()
    x = O.normal_tensor(8, (64, 48), 1.0, torch.bfloat16)
    # +-Inf in the data: amax = Inf, the literal scale formula gives 1/old = 1.0, Inf saturates
    xi = x.clone()
    xi[3, 4] = float("inf")
    xi[9, 1] = -float("inf")
    want = O.quantise_current(xi, fmt)
    got = FP8Tensor(xi.cuda(), _dt(fmt))
    assert got.fp8_meta.amax.item() == float("inf") and got.fp8_meta.scale.item() == want.scale.item() == 1.0
    assert torch.equal(got.cpu().as_subclass(torch.Tensor), want.q)
    # NaN in the data: amax = NaN, scale held at 1.0, NaN bytes are sign|0x7F
    xn = x.clone()
    xn[0, 0] = float("nan")
    xn[5, 7] = torch.tensor([-64], dtype=torch.int16).view(torch.bfloat16)[0]  # 0xffc0 = -NaN
    want = O.quantise_current(xn, fmt)
    got = FP8Tensor(xn.cuda(), _dt(fmt))
    assert math.isnan(got.fp8_meta.amax.item()) and got.fp8_meta.scale.item() == 1.0
    q = got.cpu().as_subclass(torch.Tensor)
    assert torch.equal(q, want.q) and q[0, 0] == 0x7F and q[5, 7] == 0xFF
    # all zeros: amax 0, scale held at 1.0
    z = torch.zeros(33, 9, dtype=torch.float16)
    z[2, 2] = -0.0
    got = FP8Tensor(z.cuda(), _dt(fmt))
    assert got.fp8_meta.amax.item() == 0.0 and got.fp8_meta.scale.item() == 1.0
    assert torch.equal(got.cpu().as_subclass(torch.Tensor), O.quantise_current(z, fmt).q)
    # tiny amax: quotient overflows, scale = +Inf (kept literal), bytes follow the oracle except the
    # sign of NaNs generated by 0*Inf, which no specification fixes
    t = torch.full((16,), 1e-38, dtype=torch.float32)
    got = FP8Tensor(t.cuda(), _dt(fmt))
    assert math.isinf(got.fp8_meta.scale.item())
    assert torch.equal(got.cpu().as_subclass(torch.Tensor), O.quantise_current(t, fmt).q)
    with pytest.raises(RuntimeError):
        FP8Tensor(torch.empty(0, 4, device="cuda"), _dt(fmt))


@pytest.mark.parametrize("fmt", FMTS)
def test_amax_scale_entry_point_and_fp32_near_power_of_two(fmt):
    nt, *_ = _api()
    f = nt.E4M3 if fmt == O.E4M3 else nt.E5M2
    ws = nt.workspace(torch.device("cuda", 0))
    out = torch.zeros(2, dtype=torch.float32, device="cuda")
    ks = torch.arange(-20, 21, dtype=torch.float32)
    p = torch.pow(torch.tensor(2.0), ks)
    cases = []
    for d in (-2, -1, 0, 1):
        cases += (torch.tensor(O.FP8_MAX[fmt]) / (p.view(torch.int32) + d).view(torch.float32)).tolist()
    for a in cases:
        x = torch.full((37,), a / 3, dtype=torch.float32)
        x[11] = -a
        xg = x.cuda()
        nt.check(nt.lib.ntfp8_amax_scale(xg.data_ptr(), nt.F32, 37, f, 0, None, out[0:].data_ptr(), out[1:].data_ptr(),
                                         ws.data_ptr(), nt.stream_ptr(xg.device)), "amax_scale")
        am, sc = out.tolist()
        assert am == np.float32(a)
        assert sc == O.update_scaling_factor(torch.tensor(a, dtype=torch.float32), torch.tensor(1.0), fmt).item(), a
    assert int(ws.abs().sum()) == 0, "workspace must be left zeroed"


@pytest.mark.parametrize("fmt", FMTS)
def test_update_scaling_factor_device_exhaustive_bf16(fmt):
    *_, T = _api()
    bits = torch.arange(0, 0x8000, dtype=torch.int32).to(torch.int16)
    vals = bits.view(torch.bfloat16).float()
    for old in (1.0, 3.0):
        for margin in (0, 1):
            want = O.update_scaling_factor(vals, torch.full_like(vals, old), fmt, margin)
            got = T.update_scaling_factor(vals.cuda(), torch.tensor(old, device="cuda"), _dt(fmt), margin).cpu()
            assert torch.equal(want.view(torch.int32), got.view(torch.int32))
    g = torch.Generator().manual_seed(7)
    a = torch.exp(torch.rand(300_000, generator=g) * 170 - 85).float()
    want = O.update_scaling_factor(a, torch.ones_like(a), fmt)
    got = T.update_scaling_factor(a.cuda(), torch.ones(1, device="cuda").expand_as(a), _dt(fmt)).cpu()
    assert torch.equal(want.view(torch.int32), got.view(torch.int32))


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(128, 128), (384, 256), (100, 36), (16, 200), (129, 128)])
def test_fused_transposed_output(fmt, dtype, shape):
    _, _, _, FP8Tensor, _ = _api()
    x = O.normal_tensor(17, shape, 1.0, dtype)
    x[1, 2] = float("nan")
    want = O.quantise_current(x, fmt)
    got = FP8Tensor(x.cuda(), _dt(fmt), with_transpose=True)
    assert torch.equal(got.cpu().as_subclass(torch.Tensor), want.q)
    t = got.transposed()
    assert t.shape == (shape[1], shape[0]) and t.fp8_meta is got.fp8_meta
    assert torch.equal(t.cpu().as_subclass(torch.Tensor), O.fp8_transpose(want.q))
    # the stand-alone transpose kernel (tex.fp8_transpose counterpart)
    plain = FP8Tensor(x.cuda(), _dt(fmt))
    assert torch.equal(plain.transposed().cpu().as_subclass(torch.Tensor), O.fp8_transpose(want.q))


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("with_t", [False, True])
def test_delayed_scaling_outlier_stream_small(fmt, with_t):
    _, _, DelayedScaling, FP8Tensor, _ = _api()
    st = DelayedScaling(_dt(fmt), history_len=16)
    ref = O.DelayedScaling(fmt, history_len=16)
    for step in range(24):
        x = O.student_t_outlier_tensor(2000 + step, (256, 384))
        if step == 13:
            x[0, 0] = float("nan")
        want = ref.quantise(x)
        got = FP8Tensor(x.cuda(), _dt(fmt), state=st, with_transpose=with_t)
        assert same_float(got.fp8_meta.amax.item(), want.amax.item()), step
        assert got.fp8_meta.scale.item() == want.scale.item(), step
        assert st.scale.item() == ref.scale.item(), step
        h, hr = st.amax_history.cpu(), ref.hist
        assert torch.equal(torch.isnan(h), torch.isnan(hr)) and torch.equal(h.nan_to_num(-1), hr.nan_to_num(-1)), step
        assert torch.equal(got.cpu().as_subclass(torch.Tensor), want.q), step
        if with_t:
            assert torch.equal(got.transposed().cpu().as_subclass(torch.Tensor), O.fp8_transpose(want.q)), step
        assert st.initialised == ref.initialised


@pytest.mark.parametrize("fmt", FMTS)
def test_delayed_scaling_zero_first_then_values(fmt):
    _, _, DelayedScaling, FP8Tensor, _ = _api()
    st = DelayedScaling(_dt(fmt), history_len=3, margin=1)
    ref = O.DelayedScaling(fmt, history_len=3, margin=1)
    seq = [torch.zeros(40, 24), torch.full((40, 24), 2.0), torch.full((40, 24), 900.0), torch.full((40, 24), 0.01)] * 2
    for i, x in enumerate(seq):
        x = x.to(torch.bfloat16)
        want = ref.quantise(x)
        got = FP8Tensor(x.cuda(), _dt(fmt), state=st)
        assert got.fp8_meta.scale.item() == want.scale.item(), i
        assert st.scale.item() == ref.scale.item(), i
        assert torch.equal(st.amax_history.cpu(), ref.hist), i
        q = got.cpu().as_subclass(torch.Tensor)
        assert torch.equal(q, want.q), i
        if i in (2, 6):  # 900.0 cast with the stale scale of the 2.0 step: clipped to +max
            assert int(q[0, 0]) == (0x7E if fmt == O.E4M3 else 0x7B)


@pytest.mark.parametrize("fmt", FMTS)
def test_first_use_entry_point_decides_on_the_device(fmt):
    """ntfp8_quantize_first_use: a role without a scale is scaled from its own amax (src/nanotron/fp8/tensor.py:25-28),
    a role with one casts with it, and which of the two it is is a flag in device memory that the kernels read and set
    themselves.  A sequence that holds the flag down for three steps (zeros, NaN, Inf) and then sets it, every step
    against the oracle's state machine bit for bit, without the host reading anything in between."""
    from nanotron_amd import _native as nt

    dev = torch.device("cuda")
    H = 4
    state = torch.zeros(1 + H, device=dev)
    state[0] = 1.0
    flag = torch.zeros(1, device=dev)
    ref = O.DelayedScaling(fmt, history_len=H, margin=0)
    g = torch.Generator().manual_seed(5)
    seq = [torch.zeros(48, 80), torch.full((48, 80), float("nan")), torch.full((48, 80), float("inf")),
           torch.randn(48, 80, generator=g) * 3, torch.randn(48, 80, generator=g) * 300, torch.zeros(48, 80),
           torch.randn(48, 80, generator=g) * 0.01, torch.randn(48, 80, generator=g)]
    seq[2][1:] = 1.0
    results = []
    ws, st = nt.workspace_and_stream(dev)
    for x in seq:
        xg = x.to(torch.bfloat16).to(dev)
        out = torch.empty(48, 80, dtype=torch.uint8, device=dev)
        sc = torch.empty(2, device=dev)
        nt.check(nt.lib.ntfp8_quantize_first_use(xg.data_ptr(), nt.BF16, 48, 80, nt.E4M3 if fmt == O.E4M3 else nt.E5M2, 0,
                                                 state.data_ptr(), state.data_ptr() + 4, H, flag.data_ptr(), sc.data_ptr(),
                                                 sc.data_ptr() + 4, out.data_ptr(), None, ws.data_ptr(), st), "first_use")
        results.append((xg, out, sc, state.clone(), flag.clone()))
    for i, (x, (xg, out, sc, stt, fl)) in enumerate(zip(seq, results)):
        want = ref.quantise(x.to(torch.bfloat16))
        assert same_float(sc[0].item(), want.amax.item()), i
        assert sc[1].item() == want.scale.item(), i
        assert stt[0].item() == ref.scale.item(), i
        h, hr = stt[1:].cpu(), ref.hist
        assert torch.equal(torch.isnan(h), torch.isnan(hr)) and torch.equal(h.nan_to_num(-1), hr.nan_to_num(-1)), i
        assert torch.equal(out.cpu(), want.q), i
        assert bool(fl.item() != 0) == ref.initialised, i


@pytest.mark.parametrize("fmt", FMTS)
def test_config2_full_size_20_steps(fmt):
    """Benchmark config 2: bf16 [4096,4096] Student-t + outliers, history 16, 20 steps."""
    _, _, DelayedScaling, FP8Tensor, _ = _api()
    st = DelayedScaling(_dt(fmt), history_len=16)
    ref = O.DelayedScaling(fmt, history_len=16)
    for step in range(20):
        x = O.student_t_outlier_tensor(1234 + 100 * 2 + step, (4096, 4096))
        want = ref.quantise(x)
        got = FP8Tensor(x.cuda(), _dt(fmt), state=st)
        assert got.fp8_meta.amax.item() == want.amax.item(), step
        assert got.fp8_meta.scale.item() == want.scale.item(), step
        assert st.scale.item() == ref.scale.item(), step
        assert torch.equal(st.amax_history.cpu(), ref.hist), step
        q = got.cpu().as_subclass(torch.Tensor)
        assert torch.equal(q, want.q), step


# ------------------------------------------------------------------ the reference's own tests, mirrored
@pytest.mark.parametrize("size", [4, 8, 16, 64])
def test_quantize_and_dequantize_tensor_in_fp8(size):
    # tests/fp8/test_tensor.py:13-39
    from nanotron_amd.fp8 import DTypes, FP8Tensor
    from nanotron_amd.fp8.dtypes import DType
    from nanotron_amd.fp8.meta import FP8Meta
    from nanotron_amd.fp8.tensor import convert_tensor_from_fp8

    tensor = torch.randn((size, size), dtype=torch.float32, device="cuda")
    ref_tensor = tensor.detach().clone()
    fp8_tensor = FP8Tensor(tensor, dtype=DTypes.FP8E4M3)
    assert isinstance(fp8_tensor, FP8Tensor)
    assert isinstance(fp8_tensor.fp8_meta, FP8Meta)
    assert fp8_tensor.device == ref_tensor.device
    assert fp8_tensor.dtype == torch.uint8
    assert fp8_tensor.shape == ref_tensor.shape
    assert fp8_tensor.numel() == ref_tensor.numel()
    assert not np.array_equal(fp8_tensor.cpu().numpy(), ref_tensor.cpu().numpy())
    assert fp8_tensor.fp8_meta.amax == ref_tensor.abs().max()
    assert isinstance(fp8_tensor.fp8_meta.inverse_scale, torch.Tensor)
    assert fp8_tensor.fp8_meta.scale != 0.1 and fp8_tensor.fp8_meta.scale != 1
    assert isinstance(fp8_tensor.fp8_meta.te_dtype, DType)
    tensor = convert_tensor_from_fp8(fp8_tensor, fp8_tensor.fp8_meta, torch.float32)
    assert isinstance(tensor, torch.Tensor)
    assert tensor.dtype == ref_tensor.dtype
    assert torch.allclose(tensor, ref_tensor, rtol=1e-1, atol=1e-1)


def test_fp8_tensor_attrs():
    # tests/fp8/test_tensor.py:42-55
    from nanotron_amd.fp8 import DTypes, FP8Tensor
    from nanotron_amd.fp8.meta import FP8Meta

    tensor = torch.randn((64, 64), dtype=torch.float32, device="cuda:0")
    ref_tensor = tensor.detach().clone()
    fp8_tensor = FP8Tensor(tensor, DTypes.FP8E4M3)
    assert isinstance(fp8_tensor, FP8Tensor)
    assert isinstance(fp8_tensor.fp8_meta, FP8Meta)
    assert fp8_tensor.device == ref_tensor.device
    assert fp8_tensor.dtype == torch.uint8
    assert fp8_tensor.shape == ref_tensor.shape
    assert fp8_tensor.numel() == ref_tensor.numel()
    repr(fp8_tensor)


def test_create_fp8_parameter():
    # tests/fp8/test_fp8_parameter.py:6-17
    from nanotron_amd.fp8 import DTypes, FP8Parameter, FP8Tensor
    from nanotron_amd.fp8.meta import FP8Meta

    tensor = torch.randn(16, 16, device="cuda", dtype=torch.float32)
    fp8_parameter = FP8Parameter(tensor, DTypes.FP8E4M3)
    assert isinstance(fp8_parameter.data, FP8Tensor)
    assert fp8_parameter.requires_grad is True
    assert fp8_parameter.grad is None
    assert isinstance(fp8_parameter.fp8_meta, FP8Meta)
    assert isinstance(fp8_parameter.data.fp8_meta, FP8Meta)
    repr(fp8_parameter)


def test_convert_tensor_to_fp8_with_given_meta():
    from nanotron_amd.fp8 import DTypes
    from nanotron_amd.fp8.meta import FP8Meta
    from nanotron_amd.fp8.tensor import convert_tensor_to_fp8

    x = O.normal_tensor(3, (50, 20), 2.0, torch.float32)
    meta = FP8Meta(torch.tensor(8.0, device="cuda"), torch.tensor(32.0, device="cuda"), DTypes.FP8E5M2)
    got = convert_tensor_to_fp8(x.cuda(), meta).cpu()
    assert torch.equal(got, O.cast_to_fp8(x, torch.tensor(32.0), O.E5M2))


def test_batched_delayed_quantise_equals_the_separate_calls():
    """ntfp8_quantize_delayed_batch: tensors of one source type without a transposed copy share a launch, the rest go
    out one by one; bytes, transposed bytes, amax, scale used, next scale and history equal the separate calls."""
    from nanotron_amd.fp8 import DelayedScaling, DTypes, FP8Tensor
    from nanotron_amd.fp8.tensor import quantize_delayed_batch

    shapes = [(512, 384), (1000, 37), (128, 256), (4096, 1024), (3, 5), (256, 128), (777,), (2048, 2048)]
    dtypes = [torch.bfloat16, torch.bfloat16, torch.float32, torch.bfloat16, torch.float16, torch.bfloat16, torch.float32,
              torch.bfloat16]
    with_t = [False, False, False, False, False, True, False, True]
    tensors, states, twins = [], [], []
    for i, (shape, dt) in enumerate(zip(shapes, dtypes)):
        x = O.normal_tensor(900 + i, shape, 0.3 * (i + 1), dt)
        if i == 3:
            x[17, 5] = float("nan")   # a NaN tensor: NaN amax, scale held
        tensors.append(x.cuda())
        st = DelayedScaling(DTypes.FP8E4M3, history_len=4 + i, device="cuda")
        st._buf[0] = float(2.0 ** (i - 2))
        st._buf[1:3] = torch.tensor([0.5 * i, 3.0])
        st.initialised = True
        tw = DelayedScaling(DTypes.FP8E4M3, history_len=4 + i, device="cuda")
        tw._buf.copy_(st._buf)
        tw.initialised = True
        states.append(st)
        twins.append(tw)
    for step in range(2):   # the second step runs on the scales the first one left
        got = quantize_delayed_batch(tensors, DTypes.FP8E4M3, states, with_t)
        for x, q, st, tw, wt in zip(tensors, got, states, twins, with_t):
            want = FP8Tensor(x, DTypes.FP8E4M3, state=tw, with_transpose=wt)
            assert q.shape == x.shape
            assert torch.equal(q.as_subclass(torch.Tensor), want.as_subclass(torch.Tensor))
            if wt:
                assert torch.equal(q.transposed().as_subclass(torch.Tensor), want.transposed().as_subclass(torch.Tensor))
            for a, b in ((q.fp8_meta.amax, want.fp8_meta.amax), (q.fp8_meta.scale, want.fp8_meta.scale), (st._buf, tw._buf)):
                a, b = a.float().cpu().reshape(-1), b.float().cpu().reshape(-1)
                assert bool(torch.all((a.view(torch.int32) == b.view(torch.int32)) | (a.isnan() & b.isnan())))
    from nanotron_amd import _native as nt

    pool, _ = nt.workspace_pool(torch.device("cuda", 0), 1)
    assert int(pool.abs().sum().item()) == 0, "every workspace of the pool is left zeroed"


def test_requantize_fp8_weights_batches_and_matches_per_layer_refresh():
    from torch import nn

    from nanotron_amd.fp8 import FP8Linear
    from nanotron_amd.fp8.optim import requantize_fp8_weights

    def build():
        torch.manual_seed(3)
        return nn.Sequential(FP8Linear(256, 512, bias=False, device="cuda", delayed_scaling=True, amax_history_len=4),
                             FP8Linear(512, 250, bias=False, device="cuda", delayed_scaling=True, amax_history_len=4),
                             FP8Linear(250, 64, bias=True, device="cuda", delayed_scaling=True, amax_history_len=4),
                             FP8Linear(64, 64, bias=False, device="cuda"))   # no delayed scaling: refreshed on its own
    a, b = build(), build()
    for step in range(3):   # step 0: no weight role holds a scale yet; steps 1, 2: one batched call
        with torch.no_grad():
            for m in (a, b):
                for p in m.parameters():
                    p.as_subclass(torch.Tensor).mul_(1.0 + 0.25 * (step + 1))
        assert requantize_fp8_weights(a) == 4
        for lin in b:
            lin.requantize_weight()
        for la, lb in zip(a, b):
            assert torch.equal(la.weight.data.as_subclass(torch.Tensor), lb.weight.data.as_subclass(torch.Tensor))
            ta, tb = getattr(la.weight.data, "_transposed", None), getattr(lb.weight.data, "_transposed", None)
            assert (ta is None) == (tb is None)
            if ta is not None:
                assert torch.equal(ta.as_subclass(torch.Tensor), tb.as_subclass(torch.Tensor))
            assert torch.equal(la.weight.fp8_meta.scale, lb.weight.fp8_meta.scale)
            if la.scaling is not None:
                assert torch.equal(la.scaling["weight"]._buf, lb.scaling["weight"]._buf)
    x = torch.randn(300, 256, device="cuda")
    assert torch.equal(a(x), b(x))
