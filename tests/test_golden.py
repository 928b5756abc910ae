"""Known answers of tests/golden/fp8_golden.npz (exact rational arithmetic on the definitions, written
by tests/golden/make_golden.py without importing the oracle or the package) against the CPU oracle in
both its statements, and, on the GPU, against the HIP path through the C ABI."""
import os

import numpy as np
import pytest
import torch

from oracle import c_oracle as C
from oracle import fp8_oracle as O

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp8_golden.npz"))
FMTS = [(O.E4M3, "e4m3"), (O.E5M2, "e5m2")]


def _same_f32(a: np.ndarray, b: np.ndarray) -> bool:
    """Bitwise equality of float32 arrays, any NaN matching any NaN."""
    a, b = np.asarray(a, dtype=np.float32), np.asarray(b, dtype=np.float32)
    nan = np.isnan(a) & np.isnan(b)
    return bool(np.all(nan | (a.view(np.uint32) == b.view(np.uint32))))


def _bf16_amax_values() -> torch.Tensor:
    bits = torch.from_numpy(G["scale_amax_bf16_bits"].astype(np.int32))
    return (bits << 16).view(torch.float32)


def _scale_from_exp(k: np.ndarray) -> np.ndarray:
    out = np.where(k == 32767, np.float32(np.inf), np.exp2(np.minimum(k, 127).astype(np.float64))).astype(np.float32)
    return out


# ------------------------------------------------------------------ CPU: the oracle against the golden file
@pytest.mark.parametrize("fmt,name", FMTS)
def test_oracle_decode_tables(fmt, name):
    want = G[f"decode_{name}"]
    assert _same_f32(O.decode_table(fmt), want)
    assert _same_f32(C.decode_table(fmt), want)
    assert _same_f32(O.upcast(torch.arange(256, dtype=torch.uint8), fmt).numpy(), want)


@pytest.mark.parametrize("fmt,name", FMTS)
def test_oracle_scale_for_every_bf16_amax(fmt, name):
    a = _bf16_amax_values()
    want = _scale_from_exp(G[f"scale_exp_{name}"])
    got = O.update_scaling_factor(a, torch.ones_like(a), fmt).numpy()
    assert _same_f32(got, want)
    for i in range(0, a.numel(), 97):  # the scalar statements, sampled
        assert np.float32(O.scale_closed_form(float(a[i]), 1.0, fmt)) == want[i] or (np.isinf(want[i]))
        assert np.float32(C.update_scale(float(a[i]), 1.0, fmt)) == want[i]


@pytest.mark.parametrize("fmt,name", FMTS)
def test_oracle_scale_special_values(fmt, name):
    ins, want = G["scale_special_in"], G[f"scale_special_{name}"]
    for (a, old), w in zip(ins, want):
        got = O.update_scaling_factor(torch.tensor(a), torch.tensor(old), fmt).numpy()
        assert _same_f32(got, w), (a, old, got, w)
        assert _same_f32(np.float32(O.scale_closed_form(float(a), float(old), fmt)), w)
        assert _same_f32(np.float32(C.update_scale(float(a), float(old), fmt)), w)


@pytest.mark.parametrize("fmt,name", FMTS)
def test_oracle_casts(fmt, name):
    x, s, want = G[f"cast_x_{name}"], G[f"cast_scale_{name}"], G[f"cast_bytes_{name}"]
    for sv in np.unique(s):
        sel = s == sv
        xt = torch.from_numpy(x[sel])
        assert np.array_equal(O.cast_to_fp8(xt, torch.tensor(sv), fmt).numpy(), want[sel])
        assert np.array_equal(C.cast_to_fp8(xt, float(sv), fmt).numpy(), want[sel])


@pytest.mark.parametrize("fmt,name", FMTS)
def test_oracle_delayed_scaling_sequence(fmt, name):
    ds, dc = O.DelayedScaling(fmt, history_len=4), C.DelayedScalingC(fmt, history_len=4)
    for t, a in enumerate(G["delayed_amax"]):
        x = torch.tensor([0.0, float(a), -0.0 if np.isnan(a) else -float(a) / 2], dtype=torch.float32)
        q = ds.quantise(x)
        assert _same_f32(q.scale.numpy(), G[f"delayed_used_{name}"][t])
        assert _same_f32(ds.scale.numpy(), G[f"delayed_next_{name}"][t])
        assert _same_f32(ds.hist.numpy(), G[f"delayed_hist_{name}"][t])
        _, ac, used = dc.quantise(x)
        assert _same_f32(np.float32(used), G[f"delayed_used_{name}"][t])
        assert _same_f32(np.float32(dc.scale.value), G[f"delayed_next_{name}"][t])
        assert _same_f32(dc.hist.numpy(), G[f"delayed_hist_{name}"][t])


@pytest.mark.parametrize("fa", [O.E4M3, O.E5M2])
@pytest.mark.parametrize("fb", [O.E4M3, O.E5M2])
def test_oracle_integer_gemm(fa, fb):
    a, b, want = (torch.from_numpy(G[k]) for k in ("gemm_a", "gemm_b", "gemm_d"))
    one = torch.tensor(1.0)
    aq, bq = O.cast_to_fp8(a, one, fa), O.cast_to_fp8(b, one, fb)
    assert torch.equal(O.upcast(aq, fa), a) and torch.equal(O.upcast(bq, fb), b)
    assert torch.equal(O.gemm_nt(aq, fa, one, bq, fb, one), want)
    assert torch.equal(C.gemm_nt(aq, fa, 1.0, bq, fb, 1.0), want)
    assert torch.equal(O.gemm_nt(aq, fa, torch.tensor(4.0), bq, fb, torch.tensor(0.5)), want * 0.5)


# ------------------------------------------------------------------ GPU: the HIP path against the golden file
def _dt(fmt):
    from nanotron_amd.fp8 import DTypes

    return DTypes.FP8E4M3 if fmt == O.E4M3 else DTypes.FP8E5M2


@pytest.mark.gpu
@pytest.mark.parametrize("fmt,name", FMTS)
def test_gpu_decode_and_casts(fmt, name):
    from nanotron_amd.fp8.meta import FP8Meta
    from nanotron_amd.fp8.tensor import convert_tensor_from_fp8, convert_tensor_to_fp8

    one = torch.tensor(1.0, device="cuda")
    codes = torch.arange(256, dtype=torch.uint8, device="cuda")
    dec = convert_tensor_from_fp8(codes, FP8Meta(one.clone(), one.clone(), _dt(fmt)), torch.float32).cpu().numpy()
    assert _same_f32(dec, G[f"decode_{name}"])
    x, s, want = G[f"cast_x_{name}"], G[f"cast_scale_{name}"], G[f"cast_bytes_{name}"]
    for sv in np.unique(s):
        sel = s == sv
        for dt in (torch.float32,):
            xt = torch.from_numpy(x[sel]).to(dt).cuda()
            meta = FP8Meta(one.clone(), torch.tensor(float(sv), device="cuda"), _dt(fmt))
            got = convert_tensor_to_fp8(xt, meta).cpu().numpy()
            assert np.array_equal(got, want[sel])


@pytest.mark.gpu
@pytest.mark.parametrize("fmt,name", FMTS)
def test_gpu_scale_for_every_bf16_amax_and_specials(fmt, name):
    from nanotron_amd.fp8.tensor import update_scaling_factor

    a = _bf16_amax_values().cuda()
    got = update_scaling_factor(a, torch.ones_like(a), _dt(fmt)).cpu().numpy()
    assert _same_f32(got, _scale_from_exp(G[f"scale_exp_{name}"]))
    ins = torch.from_numpy(G["scale_special_in"])
    got = update_scaling_factor(ins[:, 0].contiguous().cuda(), ins[:, 1].contiguous().cuda(), _dt(fmt)).cpu().numpy()
    assert _same_f32(got, G[f"scale_special_{name}"])
    host = update_scaling_factor(ins[:, 0].contiguous(), ins[:, 1].contiguous(), _dt(fmt)).numpy()
    assert _same_f32(host, G[f"scale_special_{name}"])


@pytest.mark.gpu
@pytest.mark.parametrize("fmt,name", FMTS)
def test_gpu_delayed_scaling_sequence(fmt, name):
    from nanotron_amd.fp8 import DelayedScaling, FP8Tensor

    st = DelayedScaling(_dt(fmt), history_len=4, device="cuda")
    for t, a in enumerate(G["delayed_amax"]):
        x = torch.zeros(64, 48, dtype=torch.bfloat16)
        x[3, 5] = float(a)
        if not np.isnan(a):
            x[17, 40] = -float(a) / 2
        q = FP8Tensor(x.cuda(), _dt(fmt), state=st, with_transpose=(t % 2 == 0))
        assert _same_f32(q.fp8_meta.amax.cpu().numpy(), np.float32(a))
        assert _same_f32(q.fp8_meta.scale.cpu().numpy(), G[f"delayed_used_{name}"][t])
        assert _same_f32(st.scale.cpu().numpy(), G[f"delayed_next_{name}"][t])
        assert _same_f32(st.amax_history.cpu().numpy(), G[f"delayed_hist_{name}"][t])


@pytest.mark.gpu
@pytest.mark.parametrize("fa", [O.E4M3, O.E5M2])
@pytest.mark.parametrize("fb", [O.E4M3, O.E5M2])
def test_gpu_integer_gemm(fa, fb):
    from nanotron_amd.fp8 import FP8Tensor
    from nanotron_amd.fp8.kernel import _gemm_nt

    a, b, want = (torch.from_numpy(G[k]) for k in ("gemm_a", "gemm_b", "gemm_d"))
    aq, bq = FP8Tensor(a.cuda(), _dt(fa)), FP8Tensor(b.cuda(), _dt(fb))  # amax 4: scale 64 / 8192, exact
    assert torch.equal(_gemm_nt(aq, bq, torch.float32, None).cpu(), want)
    assert torch.equal(_gemm_nt(aq, bq, torch.bfloat16, None).cpu(), want.to(torch.bfloat16))
