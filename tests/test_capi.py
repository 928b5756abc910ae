"""CPU-side checks of the C-ABI library: it loads, exports every symbol the header declares, the
Python binding covers all of them, and argument errors are reported as codes before any launch."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ntfp8.h")


def declared_functions():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(ntfp8_[a-z0-9_]+)\s*\(", src)))


def test_library_exports_every_declared_symbol():
    from nanotron_amd import _native as nt

    names = declared_functions()
    assert len(names) >= 11
    for n in names:
        assert hasattr(nt.lib, n), f"{n} declared in include/ntfp8.h but not exported"
        assert n in nt.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(nt.SIGNATURES) == names
    assert nt.version() == 3
    assert nt.strerror(0) == "ok" and "NULL" in nt.strerror(-1)


def test_header_constants_match_binding():
    from nanotron_amd import _native as nt

    src = open(HEADER).read()
    assert int(re.search(r"#define NTFP8_WORKSPACE_BYTES (\d+)", src).group(1)) == nt.WORKSPACE_BYTES
    assert re.search(r"NTFP8_E4M3 = 0, NTFP8_E5M2 = 1", src)
    assert re.search(r"NTFP8_F32 = 0, NTFP8_F16 = 1, NTFP8_BF16 = 2", src)


def test_argument_errors_are_codes_not_faults():
    from nanotron_amd import _native as nt

    L = nt.lib
    P = 0x10000  # a non-NULL, 16-byte aligned fake pointer: never dereferenced when validation fails
    # NULL pointers
    assert L.ntfp8_gemm(None, 0, P, P, 0, P, P, 0, 16, 16, 16, 0, None) == -1
    assert L.ntfp8_cast_to_fp8(None, 2, 4, 4, P, 0, P, None, None) == -1
    assert L.ntfp8_cast_to_fp8(P, 2, 4, 4, P, 0, None, None, None) == -1
    assert L.ntfp8_quantize_delayed(P, 2, 4, 4, 0, 0, None, P, 16, P, P, P, None, P, None) == -1
    assert L.ntfp8_amax_scale(P, 2, 16, 0, 0, None, None, P, P, None) == -1
    assert L.ntfp8_transpose(None, 4, 4, P, None) == -1
    assert L.ntfp8_cast_from_fp8(P, 0, None, 16, P + 4096, 0, None) == -1
    # bad enums
    assert L.ntfp8_gemm(P, 7, P, P, 0, P, P + (1 << 20), 0, 16, 16, 16, 0, None) == -2
    assert L.ntfp8_cast_to_fp8(P, 9, 4, 4, P, 0, P + 4096, None, None) == -2
    assert L.ntfp8_cast_from_fp8(P, 0, P, 16, P + 4096, 5, None) == -2
    # sizes
    assert L.ntfp8_gemm(P, 0, P, P, 0, P, P + (1 << 20), 0, 0, 16, 16, 0, None) == -3
    assert L.ntfp8_gemm(P, 0, P, P, 0, P, P + (1 << 20), 0, 16, -1, 16, 0, None) == -3
    assert L.ntfp8_cast_to_fp8(P, 2, 0, 4, P, 0, P + 4096, None, None) == -3
    assert L.ntfp8_cast_to_fp8(P, 2, 1 << 40, 1 << 40, P, 0, P + 4096, None, None) == -3
    assert L.ntfp8_quantize_delayed(P, 2, 4, 4, 0, 0, P, P, 0, P, P, P + 4096, None, P, None) == -3
    assert L.ntfp8_quantize_delayed(P, 2, 4, 4, 0, 500, P, P, 16, P, P, P + 4096, None, P, None) == -3
    assert L.ntfp8_amax_scale(P, 2, 0, 0, 0, None, P, P, P, None) == -3
    # alignment
    assert L.ntfp8_cast_to_fp8(P + 1, 2, 4, 4, P, 0, P + 4096, None, None) == -4
    assert L.ntfp8_cast_to_fp8(P, 0, 4, 4, P + 2, 0, P + 4096, None, None) == -4
    assert L.ntfp8_gemm(P, 0, P + 1, P, 0, P, P + (1 << 20), 0, 16, 16, 16, 0, None) == -4
    # unsupported: accumulate into a 16-bit output
    assert L.ntfp8_gemm(P, 0, P, P + 4096, 0, P, P + (1 << 20), 2, 16, 16, 16, 1, None) == -5
    # aliasing
    assert L.ntfp8_cast_to_fp8(P, 2, 4, 4, P + 4096, 0, P + 8, None, None) == -7
    assert L.ntfp8_transpose(P, 4, 4, P + 8, None) == -7
    assert L.ntfp8_gemm(P, 0, P + 4096, P + 8192, 0, P + 4096, P + 64, 0, 16, 16, 16, 0, None) == -7


def test_host_scale_function_matches_oracle():
    from nanotron_amd import _native as nt
    from oracle import fp8_oracle as O

    f32 = lambda v: torch.tensor(v, dtype=torch.float32)
    for fmt, f in ((O.E4M3, nt.E4M3), (O.E5M2, nt.E5M2)):
        assert nt.update_scaling_factor_host(1.0, 1.0, f, 0) == (256.0 if fmt == O.E4M3 else 32768.0)
        bits = torch.arange(1, 0x7F80, 7, dtype=torch.int32).to(torch.int16)
        vals = bits.view(torch.bfloat16).float()
        want = O.update_scaling_factor(vals, torch.ones_like(vals), fmt)
        got = [nt.update_scaling_factor_host(v, 1.0, f, 0) for v in vals.tolist()]
        assert got == want.tolist()
        for a in (0.0, -2.0, float("nan"), float("inf"), 1e-38, 3e38):
            for m in (0, 2):
                w = O.update_scaling_factor(f32(a), f32(3.0), fmt, m).item()
                assert nt.update_scaling_factor_host(a, 3.0, f, m) == w, (a, m)
        # quotients a few ulps around powers of two
        ks = torch.arange(-20, 21, dtype=torch.float32)
        p = torch.pow(torch.tensor(2.0), ks)
        for d in (-2, -1, 0, 1):
            a = torch.tensor(O.FP8_MAX[fmt]) / (p.view(torch.int32) + d).view(torch.float32)
            w = O.update_scaling_factor(a, torch.ones_like(a), fmt).tolist()
            assert [nt.update_scaling_factor_host(v, 1.0, f, 0) for v in a.tolist()] == w


def test_python_api_surface_matches_reference_names():
    import nanotron_amd
    from nanotron_amd.fp8 import DTypes, FP8Linear, FP8Parameter, FP8Tensor  # noqa: F401
    from nanotron_amd.fp8.constants import DTYPE_TO_FP8_MAX, FP8_DTYPES, INITIAL_AMAX, INITIAL_SCALING_FACTOR
    from nanotron_amd.fp8.kernel import fp8_matmul_kernel  # noqa: F401
    from nanotron_amd.fp8.meta import FP8Meta
    from nanotron_amd.fp8.tensor import (convert_tensor_from_fp8, convert_tensor_to_fp8,  # noqa: F401
                                         convert_torch_dtype_to_te_dtype, update_scaling_factor)
    from nanotron_amd.fp8.utils import is_fp8_available

    assert [d.name for d in DTypes] == ["FP8E4M3", "FP8E5M2", "KFLOAT16"]
    assert DTYPE_TO_FP8_MAX[DTypes.FP8E4M3] == 448.0 and DTYPE_TO_FP8_MAX[DTypes.FP8E5M2] == 57344.0
    assert INITIAL_AMAX == 1.0 and INITIAL_SCALING_FACTOR == 1.0 and torch.uint8 in FP8_DTYPES
    assert convert_torch_dtype_to_te_dtype(DTypes.FP8E4M3).name == "kFloat8E4M3"
    assert convert_torch_dtype_to_te_dtype(torch.bfloat16).name == "kBFloat16"
    # update_scaling_factor on host tensors (what FP8Linear.__init__ evaluates, linear.py:33-42)
    s = update_scaling_factor(torch.tensor(1.0), torch.tensor(1.0), DTypes.FP8E4M3)
    assert s.item() == 256.0 and s.dtype == torch.float32
    assert update_scaling_factor(torch.tensor(1.0), torch.tensor(1.0), DTypes.FP8E5M2).item() == 32768.0
    with pytest.raises(ValueError):
        update_scaling_factor(torch.tensor(1.0), torch.tensor(1.0), DTypes.FP8E4M3, margin=0.5)
    m = FP8Meta(torch.tensor(2.0), torch.tensor(4.0), DTypes.FP8E4M3)
    assert m.fp8_max == 448.0 and m.inverse_scale.item() == 0.25 and m.te_dtype.name == "kFloat8E4M3"
    assert isinstance(is_fp8_available(), bool)
    # CPU construction keeps a plain nn.Parameter and falls back to F.linear (linear.py:28,53-54)
    lin = FP8Linear(8, 4, device="cpu")
    assert type(lin.weight) is torch.nn.Parameter
    x = torch.randn(3, 8, requires_grad=True)
    lin(x).sum().backward()
    assert lin.weight.grad.shape == (4, 8) and x.grad is not None
    with pytest.raises(AssertionError):
        FP8Tensor(torch.randn(4, 4), DTypes.FP8E4M3)  # CPU tensors are rejected (tensor.py:22)
    with pytest.raises(AssertionError):
        FP8Parameter(torch.randn(4, 4), DTypes.FP8E4M3)
    nanotron_amd.install_as_nanotron_fp8()
    from nanotron.fp8 import FP8Linear as RefPathLinear  # noqa
    from nanotron.fp8.tensor import update_scaling_factor as ref_path_usf  # noqa

    assert RefPathLinear is FP8Linear


def test_fp8_output_and_transposed_operand_requests_are_validated_before_any_launch():
    from nanotron_amd import _native as nt

    L = nt.lib
    P = 0x100000   # fake device pointers, never dereferenced: every call below is refused on the host

    def desc(**kw):
        d = nt.GemmDesc()
        d.A, d.scale_a, d.B, d.scale_b, d.D = P, P + (1 << 20), P + (2 << 20), P + (1 << 20) + 64, P + (3 << 20)
        d.M, d.N, d.K, d.fmt_a, d.fmt_b, d.d_dtype, d.accumulate = 256, 256, 256, 0, 0, 0, 0
        for k, v in kw.items():
            setattr(d, k, v)
        return (nt.GemmDesc * 1)(d)

    assert L.ntfp8_gemm_batch(desc(d_dtype=nt.OUT_E4M3), 1, None) == -1                                 # no scale_d
    assert L.ntfp8_gemm_batch(desc(d_dtype=nt.OUT_E5M2, scale_d=P + (4 << 20), accumulate=1), 1, None) == -5
    assert L.ntfp8_gemm_batch(desc(d_dtype=nt.OUT_E4M3, scale_d=P + (4 << 20) + 2), 1, None) == -4        # misaligned scale
    assert L.ntfp8_gemm_batch(desc(d_dtype=nt.OUT_E4M3, scale_d=P + (4 << 20), D_t=P + (3 << 20) + 64), 1, None) == -7
    # an fp8 output next to a transposed B operand is served for M a multiple of 4 only (whole words of the transposed copy)
    assert L.ntfp8_gemm_batch(desc(M=254, d_dtype=nt.OUT_E4M3, scale_d=P + (4 << 20), b_transposed=1), 1, None) == -5
    assert L.ntfp8_gemm_batch(desc(d_dtype=7), 1, None) == -2
    assert L.ntfp8_gemm(P, 0, P + (1 << 20), P + (2 << 20), 0, P + (1 << 20), P + (3 << 20), nt.OUT_E4M3, 256, 256, 256, 0, None) == -5
    # a transposed B operand outside what the kernels serve
    for m, n, k in [(256, 250, 256), (128, 256, 256), (256, 256, 128), (256, 256, 250)]:
        assert L.ntfp8_gemm_batch(desc(M=m, N=n, K=k, b_transposed=1), 1, None) == -5, (m, n, k)
    # amax bookkeeping entry point
    assert L.ntfp8_amax_finalize(None, 0, 0, P, P + 64, 16, P + 256, None, None) == -1
    assert L.ntfp8_amax_finalize(P, 5, 0, P + 4096, P + 8192, 16, P + 256, None, None) == -2
    assert L.ntfp8_amax_finalize(P, 0, 0, P + 4096, P + 8192, 0, P + 256, None, None) == -3     # history without a length
    assert L.ntfp8_amax_finalize(P, 0, 0, P + 4096, None, 4, P + 256, None, None) == -3           # length without a history
    assert L.ntfp8_amax_finalize(P, 0, 500, P + 4096, None, 0, P + 256, None, None) == -3
    assert L.ntfp8_amax_finalize(P, 0, 0, P + 4098, None, 0, P + 256, None, None) == -4
    assert ctypes.sizeof(nt.GemmDesc) == 136
    # bias: dtype, alignment, overlap with the output, not together with a transposed B operand
    B0 = P + (5 << 20)
    assert L.ntfp8_gemm_batch(desc(bias=B0, bias_dtype=7), 1, None) == -2
    assert L.ntfp8_gemm_batch(desc(bias=B0 + 2, bias_dtype=0), 1, None) == -4
    assert L.ntfp8_gemm_batch(desc(bias=P + (3 << 20) + 128, bias_dtype=2), 1, None) == -7
    assert L.ntfp8_gemm_batch(desc(bias=B0, bias_dtype=2, b_transposed=1), 1, None) == -5
    # a transposed A operand: only next to a transposed B, M a multiple of 16
    assert L.ntfp8_gemm_batch(desc(a_transposed=1), 1, None) == -5
    assert L.ntfp8_gemm_batch(desc(M=250, a_transposed=1, b_transposed=1), 1, None) == -5


def test_a_failed_batch_has_launched_nothing():
    """A problem no kernel serves is found before the first launch: the call fails as a whole, so a binder that
    falls back (transposed copy + ntfp8_gemm) never adds an accumulated gradient twice.  Proven on the host: the
    first problem's pointers are fake, so a launch of it would fault; the call must return the code instead."""
    from nanotron_amd import _native as nt

    P = 0x100000
    d = (nt.GemmDesc * 2)()
    for i, (m, n, k, bt) in enumerate([(512, 512, 512, 0), (256, 250, 256, 1)]):   # fine; transposed B with N % 16 != 0
        base = P + i * (16 << 20)
        d[i].A, d[i].scale_a, d[i].B, d[i].scale_b, d[i].D = base, base + (1 << 20), base + (2 << 20), base + (1 << 20) + 64, base + (3 << 20)
        d[i].M, d[i].N, d[i].K, d[i].fmt_a, d[i].fmt_b, d[i].d_dtype, d[i].accumulate = m, n, k, 0, 0, 0, 1 - i
        d[i].b_transposed = bt
    assert nt.lib.ntfp8_gemm_batch(d, 2, None) == -5


def test_new_entry_points_validate_on_the_host():
    from nanotron_amd import _native as nt

    L = nt.lib
    P = 0x300000
    # tex-shaped cast: amax / scale_inv bookkeeping needs the workspace
    assert L.ntfp8_te_cast_to_fp8(None, 2, 16, P, None, None, 0, P + 4096, None, None) == -1
    assert L.ntfp8_te_cast_to_fp8(P, 2, 16, P + 8192, P + 8256, None, 0, P + 4096, None, None) == -1
    assert L.ntfp8_te_cast_to_fp8(P, 2, 0, P + 8192, None, None, 0, P + 4096, None, None) == -3
    assert L.ntfp8_te_cast_to_fp8(P, 2, 16, P + 8192, P + 8258, None, 0, P + 4096, P + 16384, None) == -4
    assert L.ntfp8_te_cast_to_fp8(P, 2, 16, P + 8192, None, None, 3, P + 4096, None, None) == -2
    assert L.ntfp8_te_cast_to_fp8(P, 2, 16, P + 8192, None, None, 0, P + 8, None, None) == -7
    assert L.ntfp8_cast_from_fp8_scale_inv(P, 0, None, 16, P + 4096, 0, None) == -1
    assert L.ntfp8_cast_from_fp8_scale_inv(P, 0, P + 8192, 16, P + 4096, 9, None) == -2
    # both formats in one pass
    args = dict(x=P, x_dtype=2, n=64, margin=0, s0=P + 4096, h0=P + 4100, s1=P + 4200, h1=P + 4204, hl=16, amax=P + 4400,
                u0=None, u1=None, o0=P + 8192, o1=P + 12288, ws=P + 16384)
    call = lambda **kw: L.ntfp8_quantize_delayed_dual(*[{**args, **kw}[k] for k in args], None)
    assert call(o1=None) == -1 and call(ws=None) == -1
    assert call(n=0) == -3 and call(hl=0) == -3
    assert call(s1=P + 4202) == -4
    assert call(s1=P + 4096) == -7 and call(o1=P + 8192 + 16) == -7 and call(o0=P + 8) == -7
    # the first use of a delayed-scaling role, decided on the device
    args = dict(x=P, x_dtype=2, rows=4, cols=16, fmt=0, margin=0, state=P + 4096, hist=P + 4100, hl=16, flag=P + 4300,
                amax=P + 4400, used=P + 4404, out=P + 8192, out_t=None, ws=P + 16384)
    call = lambda **kw: L.ntfp8_quantize_first_use(*[{**args, **kw}[k] for k in args], None)
    assert call(flag=None) == -1 and call(used=None) == -1 and call(ws=None) == -1 and call(out=None) == -1
    assert call(hl=0) == -3 and call(rows=0) == -3 and call(margin=200) == -3
    assert call(fmt=2) == -2 and call(x_dtype=5) == -2
    assert call(flag=P + 4302) == -4
    assert call(out=P + 8) == -7
    # the bandwidth yardstick
    assert L.ntfp8_stream_probe(0, None, 64, P, None) == -1 and L.ntfp8_stream_probe(3, P, 64, P + 4096, None) == -2
    assert L.ntfp8_stream_probe(1, P, 48, P + 4096, None) == -3 and L.ntfp8_stream_probe(1, P + 8, 64, P + 4096, None) == -4
    assert L.ntfp8_stream_probe(2, P, 64, P + 32, None) == -7


def test_host_policy_for_transposed_copies():
    import nanotron_amd.fp8.kernel as K

    assert K.b_transposed_supported(4096, 4096, 14336) and K.b_transposed_supported(129, 144, 256)
    for m, n, k in [(4096, 4090, 4096), (128, 4096, 4096), (4096, 128, 4096), (4096, 4096, 128), (4096, 4096, 4100),
                    (4096, 1 << 20, 4096)]:
        assert not K.b_transposed_supported(m, n, k), (m, n, k)
    # a weight [out, in] is reduced over its rows in dgrad: no copy when in_features qualifies
    assert not K.needs_transposed_copy(14336, 4096) and K.needs_transposed_copy(14336, 4090) and K.needs_transposed_copy(64, 4096)
    K.READ_B_TRANSPOSED = False
    try:
        assert not K.b_transposed_supported(4096, 4096, 4096) and K.needs_transposed_copy(14336, 4096)
    finally:
        K.READ_B_TRANSPOSED = True


def test_batched_quantise_requests_are_validated_before_any_launch():
    from nanotron_amd import _native as nt

    L = nt.lib
    P = 0x200000

    def desc(k, **kw):
        d = nt.QuantDesc()
        base = P + k * (1 << 20)
        d.x, d.x_dtype, d.fmt, d.margin, d.history_len, d.rows, d.cols = base, 2, 0, 0, 16, 4, 4
        d.scale_state, d.amax_history, d.amax_out, d.out, d.workspace = base + 4096, base + 4100, base + 8192, base + 12288, base + 16384
        for name, v in kw.items():
            setattr(d, name, v)
        return d

    one = lambda d: (nt.QuantDesc * 1)(d)
    assert L.ntfp8_quantize_delayed_batch(None, 1, None) == -1
    assert L.ntfp8_quantize_delayed_batch(one(desc(0)), 0, None) == -3
    assert L.ntfp8_quantize_delayed_batch(one(desc(0)), 65, None) == -3
    assert L.ntfp8_quantize_delayed_batch(one(desc(0, workspace=None)), 1, None) == -1
    assert L.ntfp8_quantize_delayed_batch(one(desc(0, out=None)), 1, None) == -1
    assert L.ntfp8_quantize_delayed_batch(one(desc(0, x_dtype=9)), 1, None) == -2
    assert L.ntfp8_quantize_delayed_batch(one(desc(0, history_len=0)), 1, None) == -3
    assert L.ntfp8_quantize_delayed_batch(one(desc(0, rows=0)), 1, None) == -3
    assert L.ntfp8_quantize_delayed_batch(one(desc(0, scale_state=P + 4098)), 1, None) == -4
    assert L.ntfp8_quantize_delayed_batch(one(desc(0, out=P + 8)), 1, None) == -7            # output over the input
    shared = (nt.QuantDesc * 2)(desc(0), desc(1, workspace=P + 16384))                         # two tensors, one workspace
    assert L.ntfp8_quantize_delayed_batch(shared, 2, None) == -7
    shared = (nt.QuantDesc * 2)(desc(0), desc(1, scale_state=P + 4096))                        # ... or one scaling state
    assert L.ntfp8_quantize_delayed_batch(shared, 2, None) == -7


def test_static_scratch_entry_point_rejects_what_it_cannot_hold():
    """ntfp8_quantize_delayed_batch_static: more tensors than the static array has workspaces for, and every bad
    argument of the allocating variant, are refused on the host; the `workspace` members are not looked at."""
    from nanotron_amd import _native as nt

    L = nt.lib
    P = 0x400000
    src = open(HEADER).read()
    assert int(re.search(r"#define NTFP8_STATIC_MAX_TENSORS (\d+)", src).group(1)) == nt.STATIC_MAX_TENSORS

    def desc(k, **kw):
        d = nt.QuantDesc()
        base = P + k * (1 << 20)
        d.x, d.x_dtype, d.fmt, d.margin, d.history_len, d.rows, d.cols = base, 2, 0, 0, 16, 4, 4
        d.scale_state, d.amax_history, d.amax_out, d.out = base + 4096, base + 4100, base + 8192, base + 12288
        for name, v in kw.items():
            setattr(d, name, v)
        return d

    n = nt.STATIC_MAX_TENSORS + 1
    many = (nt.QuantDesc * n)(*[desc(k) for k in range(n)])
    assert L.ntfp8_quantize_delayed_batch_static(many, n, None) == -3
    assert "size" in nt.strerror(-3)
    one = lambda d: (nt.QuantDesc * 1)(d)
    assert L.ntfp8_quantize_delayed_batch_static(None, 1, None) == -1
    assert L.ntfp8_quantize_delayed_batch_static(one(desc(0)), 0, None) == -3
    assert L.ntfp8_quantize_delayed_batch_static(one(desc(0, out=None)), 1, None) == -1
    assert L.ntfp8_quantize_delayed_batch_static(one(desc(0, rows=0)), 1, None) == -3
    assert L.ntfp8_quantize_delayed_batch_static(one(desc(0, out=P + 8)), 1, None) == -7
    two = (nt.QuantDesc * 2)(desc(0), desc(1, amax_out=P + 8192))
    assert L.ntfp8_quantize_delayed_batch_static(two, 2, None) == -7


def test_tex_shim_rejects_what_it_does_not_serve_before_touching_the_gpu():
    """The Transformer-Engine-shaped binding raises RuntimeError (TE's C++ exceptions surface as that) for the forms
    it does not serve and for host tensors; no GPU is needed to get these answers."""
    import torch

    from nanotron_amd import tex_shim as tex

    e = torch.empty(0)
    a = torch.zeros(32, 32, dtype=torch.uint8)
    one = torch.ones(1)
    D = torch.empty(32, 32)

    def gemm(**kw):
        args = dict(A=a, A_scale_inverse=one, A_type=tex.DType.kFloat8E4M3, transa=True, B=a, B_scale_inverse=one,
                    B_type=tex.DType.kFloat8E4M3, transb=False, D=D, D_scale=e, D_type=tex.DType.kFloat32, D_amax=e,
                    bias=e, bias_type=tex.DType.kBFloat16, pre_gelu_out=e, grad=False, workspace=e, workspaceSize=0,
                    accumulate=False, use_split_accumulator=False, math_sm_count=0)
        args.update(kw)
        return tex.te_gemm(*args.values())

    with pytest.raises(RuntimeError, match="GELU"):
        gemm(pre_gelu_out=torch.zeros(4))
    with pytest.raises(RuntimeError, match="bias-gradient"):
        gemm(grad=True, bias=torch.zeros(32))
    with pytest.raises(RuntimeError, match="2-D"):
        gemm(A=torch.zeros(32, dtype=torch.uint8))
    with pytest.raises(RuntimeError, match="reduction lengths"):
        gemm(B=torch.zeros(32, 48, dtype=torch.uint8))
    with pytest.raises(RuntimeError, match="device tensor"):
        tex.cast_to_fp8(torch.zeros(4, 4), one, one.clone(), one.clone(), tex.DType.kFloat8E4M3)
    with pytest.raises(RuntimeError, match="device tensor"):
        tex.cast_from_fp8(a, one, tex.DType.kFloat8E4M3, tex.DType.kFloat32)
    with pytest.raises(RuntimeError, match="not an FP8 type"):
        tex.fp8_transpose(a, tex.DType.kFloat32)
    # install() registers the module under the names the reference imports
    import sys
    keep = {k: sys.modules.get(k) for k in ("transformer_engine", "transformer_engine_extensions")}
    try:
        assert tex.install() is tex and sys.modules["transformer_engine_extensions"] is tex
        assert "transformer_engine" in sys.modules
    finally:
        for k, v in keep.items():
            if v is None:
                sys.modules.pop(k, None)
            else:
                sys.modules[k] = v


def test_profiling_build_exports_its_accessors():
    """The product library carries no profiling accessors.  The profiling build (nanotron_amd/profiling/, made on request by
    `python -m nanotron_amd.build --profiling` and loaded only by bench.py --workload wg-timeline) is the product
    library plus two of them; it is checked when it is there."""
    import ctypes

    import pytest

    from nanotron_amd import _native as nt
    from nanotron_amd.build import EXPERIMENTS, LIB_STAMPS, experiment_lib

    assert not hasattr(nt.lib, "ntfp8_debug_stamps") and not hasattr(nt.lib, "ntfp8_debug_set_tile_order")
    paths = [p for p in [LIB_STAMPS] + [experiment_lib(n) for n in EXPERIMENTS] if os.path.exists(p)]
    if not paths:
        pytest.skip("no profiling build in the tree (python -m nanotron_amd.build --profiling)")
    for path in paths:
        lib = ctypes.CDLL(path)
        for name in ("ntfp8_debug_stamps", "ntfp8_debug_set_tile_order", "ntfp8_gemm_batch", "ntfp8_version"):
            assert hasattr(lib, name), (path, name)
        lib.ntfp8_debug_stamps.restype = ctypes.c_int
        lib.ntfp8_debug_stamps.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
        assert lib.ntfp8_debug_stamps(None, 64) < 0
