"""Pins the oracle (oracle/fp8_oracle.py and oracle/fp8_oracle.c) against evidence that does
not come from the oracle's own formulas: the OCP FP8 spec tables, closed forms, the known
answers the reference itself evaluates, exhaustive sweeps and two independent encoders."""
import math

import numpy as np
import pytest
import torch

from oracle import c_oracle as C
from oracle import fp8_oracle as O

FMTS = [O.E4M3, O.E5M2]


def f32(v):
    return torch.tensor(v, dtype=torch.float32)


# ----------------------------------------------------------------------------- scale
def test_scale_known_answers_from_reference_linear_init():
    # fp8/linear.py:33-42 evaluates update_scaling_factor(amax=1.0, 1.0): 448 -> 2**8, 57344 -> 2**15
    assert O.update_scaling_factor(f32(1.0), f32(1.0), O.E4M3).item() == 256.0
    assert O.update_scaling_factor(f32(1.0), f32(1.0), O.E5M2).item() == 32768.0
    assert C.update_scale(1.0, 1.0, O.E4M3) == 256.0
    assert C.update_scale(1.0, 1.0, O.E5M2) == 32768.0


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("src", ["bf16", "fp16"])
def test_scale_exhaustive_halfprecision_amax_vs_exact_exponent(fmt, src):
    bits = torch.arange(0, 0x8000, dtype=torch.int32).to(torch.int16)
    vals = bits.view(torch.bfloat16 if src == "bf16" else torch.float16).float()
    vals = vals[torch.isfinite(vals) & (vals > 0)]
    got = O.update_scaling_factor(vals, torch.full_like(vals, 1.0), fmt)
    q = (torch.tensor(O.FP8_MAX[fmt]) / vals)
    finite = torch.isfinite(q)
    # exact exponent extraction of the fp32 quotient
    _, e = torch.frexp(q[finite].double())
    want = torch.pow(torch.tensor(2.0, dtype=torch.float64), (e - 1).double()).float()
    assert torch.equal(got[finite], want)
    assert torch.all(torch.isinf(got[~finite]))
    # invariants: power of two, amax*scale <= fp8_max < 2*amax*scale
    g = got[finite].double()
    m, _ = torch.frexp(g)
    assert torch.all(m == 0.5)
    a = vals[finite].double()
    assert torch.all(a * g <= O.FP8_MAX[fmt])
    assert torch.all(2 * a * g > O.FP8_MAX[fmt])
    # C restatement and the closed form agree bit for bit on a strided subset
    for v in vals[::97].tolist():
        t = O.update_scaling_factor(f32(v), f32(1.0), fmt).item()
        assert C.update_scale(v, 1.0, fmt) == t
        assert O.scale_closed_form(v, 1.0, fmt) == t


@pytest.mark.parametrize("fmt", FMTS)
def test_scale_edge_rows(fmt):
    old = f32(3.0)
    for bad in [0.0, -1.0, float("nan")]:
        assert O.update_scaling_factor(f32(bad), old, fmt).item() == 3.0
        assert C.update_scale(bad, 3.0, fmt) == 3.0
        assert O.scale_closed_form(bad, 3.0, fmt) == 3.0
    # amax = Inf: log2(0) = -inf < 0, so the literal formula returns 1/old (== old for the
    # reference's only call pattern, old = 1.0)
    third = (1 / f32(3.0)).item()
    assert O.update_scaling_factor(f32(float("inf")), old, fmt).item() == third
    assert C.update_scale(float("inf"), 3.0, fmt) == third
    assert O.scale_closed_form(float("inf"), 3.0, fmt) == third
    assert O.update_scaling_factor(f32(float("inf")), f32(1.0), fmt).item() == 1.0
    tiny = 1e-38
    assert math.isinf(O.update_scaling_factor(f32(tiny), old, fmt).item())
    assert math.isinf(C.update_scale(tiny, 3.0, fmt))
    big = float(torch.finfo(torch.bfloat16).max)
    t = O.update_scaling_factor(f32(big), old, fmt).item()
    assert t == C.update_scale(big, 3.0, fmt) == O.scale_closed_form(big, 3.0, fmt)
    assert t == 2.0 ** math.floor(math.log2(O.FP8_MAX[fmt] / big))


@pytest.mark.parametrize("fmt", FMTS)
def test_scale_fp32_amax_random_and_near_power_of_two(fmt):
    g = torch.Generator().manual_seed(7)
    a = torch.exp(torch.rand(200_000, generator=g) * 60 - 30).float()
    # quotients 1..3 ulps below/above a power of two: the literal formula rounds log2 up
    ks = torch.arange(-20, 21, dtype=torch.float32)
    p = torch.pow(torch.tensor(2.0), ks)
    near = []
    for d in (-3, -2, -1, 0, 1, 2, 3):
        qq = (p.view(torch.int32) + d).view(torch.float32)
        near.append(torch.tensor(O.FP8_MAX[fmt]) / qq)
    a = torch.cat([a] + near)
    t = O.update_scaling_factor(a, torch.ones_like(a), fmt)
    sample = torch.cat([torch.arange(0, 200_000, 41), torch.arange(200_000, a.numel())])
    for i in sample.tolist():
        v = a[i].item()
        assert C.update_scale(v, 1.0, fmt) == t[i].item(), v
        assert O.scale_closed_form(v, 1.0, fmt) == t[i].item(), v


@pytest.mark.parametrize("fmt", FMTS)
def test_scale_integer_margin(fmt):
    for margin in (1, 2, -1):
        for v in (0.3, 1.0, 77.0, 1e-3, 6e4):
            t = O.update_scaling_factor(f32(v), f32(1.0), fmt, margin).item()
            assert t == C.update_scale(v, 1.0, fmt, margin) == O.scale_closed_form(v, 1.0, fmt, margin)
            assert t == O.update_scaling_factor(f32(v), f32(1.0), fmt, 0).item() / 2.0 ** margin


# ----------------------------------------------------------------------------- formats
@pytest.mark.parametrize("fmt", FMTS)
def test_decode_table_spec_vs_torch_vs_c(fmt):
    spec = O.decode_table(fmt)
    tor = torch.arange(256, dtype=torch.uint8).view(O.TORCH_FP8[fmt]).double().numpy()
    cc = C.decode_table(fmt).astype(np.float64)
    for other in (tor, cc):
        assert np.array_equal(np.isnan(spec), np.isnan(other))
        ok = ~np.isnan(spec)
        assert np.array_equal(spec[ok], other[ok])
        assert np.array_equal(np.signbit(spec[ok]), np.signbit(other[ok]))
    # spec constants
    if fmt == O.E4M3:
        assert spec[0x7E] == 448.0 and np.isnan(spec[0x7F]) and spec[0x01] == 2.0 ** -9 and spec[0x08] == 2.0 ** -6
    else:
        assert spec[0x7B] == 57344.0 and np.isinf(spec[0x7C]) and np.isnan(spec[0x7D]) and spec[0x01] == 2.0 ** -16


@pytest.mark.parametrize("fmt", FMTS)
def test_cast_fixed_points(fmt):
    one = f32(1.0)
    x = torch.tensor([float("nan"), -float("nan"), float("inf"), -float("inf"), 1e30, -1e30, -0.0, 0.0])
    want = {O.E4M3: [0x7F, 0xFF, 0x7E, 0xFE, 0x7E, 0xFE, 0x80, 0x00],
            O.E5M2: [0x7F, 0xFF, 0x7B, 0xFB, 0x7B, 0xFB, 0x80, 0x00]}[fmt]
    # copysign: make sure -nan really carries the sign bit
    x[1] = torch.tensor([0xFFC00000 - (1 << 32)], dtype=torch.int32).view(torch.float32)[0]
    assert O.cast_to_fp8(x, one, fmt).tolist() == want
    assert C.cast_to_fp8(x, 1.0, fmt).tolist() == want
    assert O.cast_to_fp8_search(x.numpy(), fmt).tolist() == want
    if fmt == O.E4M3:
        # RNE: 17->16, 19->20, 21->20, 23->24 ; subnormal 2^-9 -> 1, 2^-10 ties to 0, 3*2^-11 -> 1 (0.75 ulp)
        y = torch.tensor([17.0, 19.0, 21.0, 23.0, 2.0 ** -9, 2.0 ** -10, 3 * 2.0 ** -11, 3 * 2.0 ** -10])
        got = O.cast_to_fp8(y, one, fmt)
        dec = torch.tensor(O.decode_table(fmt))[got.long()].tolist()
        assert dec == [16.0, 20.0, 20.0, 24.0, 2.0 ** -9, 0.0, 2.0 ** -9, 2 * 2.0 ** -9 + 0 * 1]  # 1.5ulp ties to even=2
        assert C.cast_to_fp8(y, 1.0, fmt).tolist() == got.tolist()
        # 448..464 all saturate to 448 because the clamp happens before rounding
        z = torch.tensor([448.0, 455.9, 463.9, 464.0, 465.0, 1000.0])
        assert O.cast_to_fp8(z, one, fmt).tolist() == [0x7E] * 6
        assert C.cast_to_fp8(z, 1.0, fmt).tolist() == [0x7E] * 6


@pytest.mark.parametrize("fmt", FMTS)
def test_all_codes_round_trip(fmt):
    codes = torch.arange(256, dtype=torch.uint8)
    vals = codes.view(O.TORCH_FP8[fmt]).float()
    finite = torch.isfinite(vals)
    back = O.cast_to_fp8(vals, f32(1.0), fmt)
    assert torch.equal(back[finite], codes[finite])
    assert torch.equal(C.cast_to_fp8(vals, 1.0, fmt)[finite], codes[finite])


@pytest.mark.parametrize("fmt", FMTS)
def test_cast_exhaustive_bf16_three_encoders(fmt):
    bits = torch.arange(0, 0x10000, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.bfloat16)
    for k in list(range(-3, 16)) + [-20, 40, 100]:
        s = 2.0 ** k
        t = O.cast_to_fp8(x, f32(s), fmt)
        c = C.cast_to_fp8(x, s, fmt)
        assert torch.equal(t, c), f"torch vs C encoder, scale 2^{k}"
        with np.errstate(over="ignore", invalid="ignore"):
            y = (x.float().numpy() * np.float32(s)).astype(np.float32)
        srch = torch.from_numpy(O.cast_to_fp8_search(y, fmt))
        assert torch.equal(t, srch), f"torch vs search encoder, scale 2^{k}"


@pytest.mark.parametrize("fmt", FMTS)
def test_cast_fp32_midpoints_and_random(fmt):
    # every midpoint between adjacent finite fp8 magnitudes, +-1 fp32 ulp, must round as RNE says
    tab = O.decode_table(fmt)
    maxc = 0x7E if fmt == O.E4M3 else 0x7B
    mags = tab[: maxc + 1]
    mids = ((mags[:-1] + mags[1:]) / 2).astype(np.float32)
    assert np.array_equal(mids.astype(np.float64), (mags[:-1] + mags[1:]) / 2)  # midpoints are exact in fp32
    lo = np.nextafter(mids, np.float32(0))
    hi = np.nextafter(mids, np.float32(np.inf))
    codes = np.arange(maxc)
    want_mid = np.where(codes % 2 == 0, codes, codes + 1)
    for arr, want in ((mids, want_mid), (lo, codes), (hi, codes + 1)):
        for sgn in (1.0, -1.0):
            xx = torch.from_numpy((arr * sgn).astype(np.float32))
            w = torch.from_numpy(want.astype(np.uint8)) | (0x80 if sgn < 0 else 0)
            assert torch.equal(O.cast_to_fp8(xx, f32(1.0), fmt), w)
            assert torch.equal(C.cast_to_fp8(xx, 1.0, fmt), w)
    g = torch.Generator().manual_seed(11)
    x = torch.randn(1 << 20, generator=g) * torch.exp(torch.randn(1 << 20, generator=g) * 4)
    for s in (0.37, 1.0, 256.0, 3.1e4):
        t = O.cast_to_fp8(x, f32(s), fmt)
        assert torch.equal(t, C.cast_to_fp8(x, float(np.float32(s)), fmt))
        y = (x.numpy() * np.float32(s)).astype(np.float32)
        assert torch.equal(t, torch.from_numpy(O.cast_to_fp8_search(y, fmt)))


@pytest.mark.parametrize("fmt", FMTS)
def test_dequant_is_table_times_inverse_scale(fmt):
    q = torch.arange(256, dtype=torch.uint8)
    keep = torch.isfinite(q.view(O.TORCH_FP8[fmt]).float())
    for s in (1.0, 256.0, 2.0 ** -5):
        d = O.cast_from_fp8(q, f32(s), fmt, torch.float32)
        want = torch.tensor(O.decode_table(fmt) / s, dtype=torch.float32)
        assert torch.equal(d[keep], want[keep])
        assert torch.equal(C.cast_from_fp8(q, s, fmt)[keep], want[keep])


def test_transpose_is_a_byte_permutation():
    q = torch.arange(7 * 13, dtype=torch.uint8).reshape(7, 13)
    t = O.fp8_transpose(q)
    assert t.shape == (13, 7) and t.is_contiguous()
    assert torch.equal(t, C.transpose(q))
    for r in range(7):
        for c in range(13):
            assert t[c, r] == q[r, c]


# ----------------------------------------------------------------------------- amax
def test_amax_definition_nan_and_empty():
    x = torch.tensor([[1.0, -7.5], [3.0, 2.0]], dtype=torch.bfloat16)
    assert O.amax(x).item() == 7.5 and O.amax(x).dtype == torch.float32 and C.amax(x) == 7.5
    x[0, 0] = float("nan")
    assert math.isnan(O.amax(x).item()) and math.isnan(C.amax(x))
    x[0, 0] = -float("inf")
    assert O.amax(x).item() == float("inf") == C.amax(x)
    with pytest.raises(RuntimeError):
        O.amax(torch.empty(0))
    g = torch.Generator().manual_seed(3)
    for dt in (torch.float32, torch.float16, torch.bfloat16):
        y = torch.randn(10007, generator=g).to(dt)
        assert O.amax(y).item() == C.amax(y) == float(np.abs(y.float().numpy()).max())


# ----------------------------------------------------------------------------- GEMM
def _rand_q(shape, fmt, seed, std=1.0):
    x = O.normal_tensor(seed, shape, std)
    return O.quantise_current(x, fmt)


def test_gemm_integer_operands_exact_and_order_free():
    # operands are small integers with scale 1: every partial sum is an integer < 2^24, so
    # fp32 accumulation is exact in any order and all three evaluations agree bit for bit
    g = torch.Generator().manual_seed(5)
    a = torch.randint(-8, 9, (33, 96), generator=g).float()
    b = torch.randint(-8, 9, (17, 96), generator=g).float()
    one = f32(1.0)
    aq, bq = O.cast_to_fp8(a, one, O.E5M2), O.cast_to_fp8(b, one, O.E4M3)
    want = (a.double() @ b.double().t()).float()
    assert torch.equal(O.gemm_nt(aq, O.E5M2, one, bq, O.E4M3, one), want)
    assert torch.equal(C.gemm_nt(aq, O.E5M2, 1.0, bq, O.E4M3, 1.0), want)
    acc = torch.full((33, 17), 5.0)
    assert torch.equal(O.gemm_nt(aq, O.E5M2, one, bq, O.E4M3, one, accumulate_into=acc), want + 5)
    assert torch.equal(C.gemm_nt(aq, O.E5M2, 1.0, bq, O.E4M3, 1.0, accumulate_into=acc), want + 5)


def test_gemm_identity_and_one_hot_known_answers():
    xq = _rand_q((8, 16), O.E4M3, 1)
    eye = torch.eye(16)
    eq = O.cast_to_fp8(eye, f32(1.0), O.E4M3)
    d = O.gemm_nt(xq.q, O.E4M3, xq.scale, eq, O.E4M3, f32(1.0))
    assert torch.equal(d, O.cast_from_fp8(xq.q, xq.scale, O.E4M3, torch.float32))


def test_gemm_fp32_vs_fp64_and_c():
    xq = _rand_q((64, 256), O.E4M3, 21)
    wq = _rand_q((48, 256), O.E4M3, 22, 0.02)
    d32 = O.gemm_nt(xq.q, xq.fmt, xq.scale, wq.q, wq.fmt, wq.scale)
    d64 = O.gemm_nt(xq.q, xq.fmt, xq.scale, wq.q, wq.fmt, wq.scale, torch.float64, None, torch.float64)
    dc = C.gemm_nt(xq.q, xq.fmt, xq.scale.item(), wq.q, wq.fmt, wq.scale.item())
    assert O.rel_l2(d32, d64) < 1e-6
    assert O.rel_l2(dc, d64) < 1e-6
    # and against the un-quantised product: fp8 error only (loose, like tests/fp8/test_linear.py:25)
    x = O.normal_tensor(21, (64, 256), 1.0).float()
    w = O.normal_tensor(22, (48, 256), 0.02).float()
    assert O.rel_l2(d32, x @ w.t()) < 0.06


def test_fp8_matmul_kernel_operator_meaning():
    # D = op_b(B) . op_a(A)   (fp8/kernel.py:43-68)
    X = _rand_q((12, 32), O.E4M3, 31)
    W = _rand_q((20, 32), O.E4M3, 32, 0.02)
    G = _rand_q((12, 20), O.E5M2, 33, 1e-3)
    x, w, g = (O.cast_from_fp8(t.q, t.scale, t.fmt, torch.float64) for t in (X, W, G))
    y = O.linear_forward(X, W)
    assert y.shape == (12, 20) and O.rel_l2(y, x @ w.t()) < 1e-6
    dx = O.linear_dgrad(G, W)
    assert dx.shape == (12, 32) and O.rel_l2(dx, g @ w) < 1e-6
    dw = O.linear_wgrad(G, X)
    assert dw.shape == (20, 32) and O.rel_l2(dw, g.t() @ x) < 1e-6
    acc = torch.ones(20, 32)
    assert O.rel_l2(O.linear_wgrad(G, X, accumulate_into=acc), g.t() @ x + 1) < 1e-6


# ----------------------------------------------------------------------------- delayed scaling
@pytest.mark.parametrize("fmt", FMTS)
def test_delayed_scaling_known_answer_sequences(fmt):
    H = 4
    st = O.DelayedScaling(fmt, history_len=H)
    k0 = 8 if fmt == O.E4M3 else 15  # scale for amax == 1 is 2**k0
    seq = [1.0, 3.0, 0.5, 0.5, 0.5, 0.5, 0.5, float("nan"), 0.25]
    used, nxt, hists = [], [], []
    for a in seq:
        x = torch.tensor([a, -a / 2, 0.0], dtype=torch.bfloat16)
        r = st.quantise(x)
        used.append(r.scale.item())
        nxt.append(st.scale.item())
        hists.append(st.hist.clone())
    # step 0: first use -> current scaling from amax 1.0; later steps use the previous "next"
    assert used[0] == 2.0 ** k0
    assert used[1:] == nxt[:-1]
    # next scale follows max(hist): 1 -> 2^k0 ; 3 -> 2^(k0-1) (held while the 3.0 is in the window of 4)
    assert nxt[:5] == [2.0 ** k0, 2.0 ** (k0 - 1), 2.0 ** (k0 - 1), 2.0 ** (k0 - 1), 2.0 ** (k0 - 1)]
    assert nxt[5] == 2.0 ** (k0 + 1)  # 3.0 rolled out, window is all 0.5
    assert nxt[6] == 2.0 ** (k0 + 1)
    assert nxt[7] == nxt[6] and math.isnan(hists[7][0].item())  # NaN amax: scale held
    assert nxt[8] == nxt[7]  # NaN still in the window
    assert hists[2].tolist() == [0.5, 3.0, 1.0, 0.0]


@pytest.mark.parametrize("fmt", FMTS)
def test_delayed_scaling_python_vs_c_on_outlier_stream(fmt):
    st = O.DelayedScaling(fmt, history_len=16)
    sc = C.DelayedScalingC(fmt, 16)
    for step in range(20):
        x = O.student_t_outlier_tensor(1000 + step, (64, 512))
        r = st.quantise(x)
        q, a, s = sc.quantise(x)
        assert torch.equal(r.q, q) and r.amax.item() == a and r.scale.item() == s
        assert torch.equal(st.hist, sc.hist) and st.scale.item() == sc.scale.value
    # zero tensor first: stays un-initialised, scale held at 1.0
    st = O.DelayedScaling(fmt, history_len=3)
    sc = C.DelayedScalingC(fmt, 3)
    z = torch.zeros(8, dtype=torch.bfloat16)
    r = st.quantise(z)
    q, a, s = sc.quantise(z)
    assert r.scale.item() == s == 1.0 and not st.initialised and sc.init.value == 0
    x = torch.full((8,), 2.0, dtype=torch.bfloat16)
    r = st.quantise(x)
    q, a, s = sc.quantise(x)
    assert r.scale.item() == s == O.update_scaling_factor(f32(2.0), f32(1.0), fmt).item()


def test_current_scaling_step0_equals_reference_path():
    x = O.normal_tensor(9, (32, 32), 1.0, torch.float32)
    r = O.quantise_current(x, O.E4M3)
    st = O.DelayedScaling(O.E4M3)
    d = st.quantise(x)
    assert torch.equal(r.q, d.q) and r.scale.item() == d.scale.item() and r.amax.item() == x.abs().max().item()
    # tests/fp8/test_tensor.py:39 round trip at rtol=atol=0.1
    back = O.cast_from_fp8(r.q, r.scale, O.E4M3, torch.float32)
    assert torch.allclose(back, x, rtol=0.1, atol=0.1)
