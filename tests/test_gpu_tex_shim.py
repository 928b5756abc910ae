"""GPU parity of the Transformer-Engine-shaped binding (`nanotron_amd.tex_shim`): the four `tex.*` functions are
called with exactly the argument lists of the reference's call sites (src/nanotron/fp8/tensor.py:60-74,
src/nanotron/fp8/kernel.py:22-68) and compared with the CPU oracle.  Nothing of the reference is imported: the call
sites are restated below, line by line, with `tex` bound to the shim."""
import pytest
import torch

from oracle import fp8_oracle as O

pytestmark = pytest.mark.gpu


def _tex():
    from nanotron_amd import tex_shim

    return tex_shim


def _te_dtype(fmt):
    tex = _tex()
    return tex.DType.kFloat8E4M3 if fmt == O.E4M3 else tex.DType.kFloat8E5M2


def _bits(t):
    return t.detach().float().cpu().contiguous().view(torch.int32)


class _Meta:
    """The fields of the reference's FP8Meta that its call sites read (src/nanotron/fp8/meta.py:12-40)."""

    def __init__(self, amax, scale, fmt):
        self.amax, self.scale, self.fmt = amax, scale, fmt

    @property
    def te_dtype(self):
        return _te_dtype(self.fmt)

    @property
    def inverse_scale(self):
        return 1 / self.scale   # meta.py:36-37


def ref_convert_tensor_to_fp8(tensor, meta):
    """src/nanotron/fp8/tensor.py:60-65, with `tex` = the shim."""
    tex = _tex()
    inverse_scale = torch.tensor(1.0, device=tensor.device, dtype=torch.float32)
    return tex.cast_to_fp8(tensor, meta.scale, meta.amax, inverse_scale, meta.te_dtype), inverse_scale


def ref_convert_tensor_from_fp8(tensor, meta, dtype):
    """src/nanotron/fp8/tensor.py:68-74."""
    tex = _tex()
    out_t = {torch.float32: tex.DType.kFloat32, torch.float16: tex.DType.kFloat16, torch.bfloat16: tex.DType.kBFloat16}[dtype]
    return tex.cast_from_fp8(tensor, meta.inverse_scale, meta.te_dtype, out_t)


def ref_fp8_matmul_kernel(mat_a, meta_a, transpose_a, mat_b, meta_b, transpose_b, use_split_accumulator, bias=None):
    """src/nanotron/fp8/kernel.py:22-70: same statements, same 21 te_gemm arguments in the same order."""
    tex = _tex()
    device = mat_a.device
    _empty_tensor = torch.Tensor()
    # (the reference allocates [mat_a.shape[0], mat_b.shape[1]], right for its square tests only; the true shape here)
    mat_a_ = tex.fp8_transpose(mat_a, meta_a.te_dtype) if transpose_a is False else mat_a      # kernel.py:43
    mat_b_ = tex.fp8_transpose(mat_b, meta_b.te_dtype) if transpose_b is True else mat_b       # kernel.py:44
    output = torch.empty(mat_b_.shape[0], mat_a_.shape[0], device=device, dtype=torch.float32)
    workspace = torch.empty(33_554_432, dtype=torch.int8, device=device)
    accumulate = False
    out_dtype = getattr(tex.DType, "kFloat32")
    bias = torch.tensor([], dtype=torch.float32) if bias is None else bias
    TE_CONFIG_TRANSPOSE_BIAS = False
    TE_CONFIG_TRANSPOSE_A = True
    TE_CONFIG_TRANSPOSE_B = False
    SCALE = AMAX = _empty_tensor
    tex.te_gemm(
        mat_a_, meta_a.inverse_scale, meta_a.te_dtype, TE_CONFIG_TRANSPOSE_A,
        mat_b_, meta_b.inverse_scale, meta_b.te_dtype, TE_CONFIG_TRANSPOSE_B,
        output, SCALE, out_dtype, AMAX, bias, out_dtype, _empty_tensor, TE_CONFIG_TRANSPOSE_BIAS,
        workspace, workspace.shape[0], accumulate, use_split_accumulator, 0,
    )
    return output


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_cast_to_fp8_as_the_reference_calls_it(fmt, dtype):
    """tensor.py:25-28 + 60-65: amax, scale from it, cast; TE also keeps amax = max(amax, max|x|) and writes
    scale_inv = 1 / scale into the tensor it is handed."""
    x = O.normal_tensor(3, (257, 130), 3.0, dtype)
    q = O.quantise_current(x, fmt)
    xg = x.cuda()
    meta = _Meta(xg.abs().max().float().clone(), q.scale.cuda(), fmt)       # tensor.py:25-27
    got, inv = ref_convert_tensor_to_fp8(xg, meta)
    assert got.dtype == torch.uint8 and got.shape == x.shape
    assert torch.equal(got.cpu(), q.q)
    assert torch.equal(_bits(meta.amax), _bits(q.amax))                      # no-op: it already was the maximum
    assert torch.equal(_bits(inv), _bits(1 / q.scale))
    # a running amax below / above this tensor's, and a scale that is no power of two
    s = torch.tensor(3.3, device="cuda")
    for start in (0.0, 1e6):
        amax = torch.tensor(start, device="cuda")
        inv = torch.zeros((), device="cuda")
        got = _tex().cast_to_fp8(xg, s, amax, inv, _te_dtype(fmt))
        assert torch.equal(got.cpu(), O.cast_to_fp8(x, s.cpu(), fmt))
        assert amax.item() == max(start, O.amax(x).item())
        assert torch.equal(_bits(inv), _bits(1 / s.cpu()))


def test_cast_to_fp8_nan_inf_and_empty():
    tex = _tex()
    x = torch.tensor([[1.0, float("nan"), -float("inf"), 0.0, -0.0, 1e30, -3.0, 500.0]] * 5, dtype=torch.float32)
    s = torch.tensor(2.0)
    amax = torch.zeros((), device="cuda")
    inv = torch.zeros((), device="cuda")
    got = tex.cast_to_fp8(x.cuda(), s.cuda(), amax, inv, tex.DType.kFloat8E4M3)
    assert torch.equal(got.cpu(), O.cast_to_fp8(x, s, O.E4M3))
    assert torch.isnan(amax).item() and inv.item() == 0.5
    assert tex.cast_to_fp8(torch.empty(0, 4, device="cuda"), s.cuda(), amax, inv, tex.DType.kFloat8E4M3).shape == (0, 4)
    with pytest.raises(RuntimeError):
        tex.cast_to_fp8(x.cuda(), s.cuda(), amax, inv, tex.DType.kFloat32)


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_cast_from_fp8_takes_the_inverse_scale(fmt, out_dtype):
    codes = torch.arange(256, dtype=torch.uint8).repeat(3)
    for scale in (256.0, 0.125, 3.3):   # powers of two, and a scale whose reciprocal is rounded
        sc = torch.tensor(scale)
        meta = _Meta(None, sc.cuda(), fmt)
        got = ref_convert_tensor_from_fp8(codes.cuda(), meta, out_dtype).cpu()
        want = O.cast_from_fp8(codes, sc, fmt, out_dtype)
        assert got.dtype == out_dtype
        same = (got.float().view(torch.int32) == want.float().view(torch.int32)) | (got.isnan() & want.isnan())
        assert bool(same.all()), (fmt, out_dtype, scale)


def test_fp8_transpose():
    tex = _tex()
    q = torch.randint(0, 256, (300, 130), dtype=torch.uint8)
    got = tex.fp8_transpose(q.cuda(), tex.DType.kFloat8E4M3)
    assert got.is_contiguous() and torch.equal(got.cpu(), O.fp8_transpose(q))


@pytest.mark.parametrize("shape", [(16, 16, 16), (256, 384, 512), (2048, 1024, 1024), (100, 36, 52)])
def test_the_three_gemms_of_a_linear_layer_through_the_reference_call_site(shape):
    """linear.py:82-84 forward and the backward GEMMs the docstring at linear.py:92-96 states, issued through
    kernel.py's statements with inverse scales, against the oracle."""
    M, K, N = shape
    x, w, gy = O.normal_tensor(1, (M, K), 1.0), O.normal_tensor(2, (N, K), 0.02), O.normal_tensor(3, (M, N), 1e-3)
    xq, wq, gq = O.quantise_current(x, O.E4M3), O.quantise_current(w, O.E4M3), O.quantise_current(gy, O.E5M2)
    dev = lambda q: (q.q.cuda(), _Meta(q.amax.cuda(), q.scale.cuda(), q.fmt))
    (xb, xm), (wb, wm), (gb, gm) = dev(xq), dev(wq), dev(gq)
    y = ref_fp8_matmul_kernel(wb, wm, True, xb, xm, False, False)
    assert y.shape == (M, N) and O.rel_l2(y.cpu(), O.linear_forward(xq, wq)) <= 1e-3
    dx = ref_fp8_matmul_kernel(wb, wm, False, gb, gm, False, True)
    assert dx.shape == (M, K) and O.rel_l2(dx.cpu(), O.linear_dgrad(gq, wq)) <= 1e-3
    dw = ref_fp8_matmul_kernel(xb, xm, False, gb, gm, True, True)
    assert dw.shape == (N, K) and O.rel_l2(dw.cpu(), O.linear_wgrad(gq, xq)) <= 1e-3


def test_te_gemm_integer_operands_bit_exact_all_arguments():
    """Integer-valued operands sum exactly in any order: the result must equal the fp64 product bit for bit, with
    inverse scales that are no powers of two, a bias, accumulation into D, and all four transa / transb forms on
    shapes the big kernel serves in place (1024 x 512 x 256), ragged ones (300 x 272 x 384) and small ones."""
    tex = _tex()
    g = torch.Generator().manual_seed(5)
    one = torch.tensor(1.0)
    for M, N, K in [(300, 272, 384), (64, 48, 32), (1024, 512, 256)]:
        a = torch.randint(-4, 5, (N, K), generator=g).float()      # te_gemm's A: [N, K]
        b = torch.randint(-4, 5, (M, K), generator=g).float()      # te_gemm's B: [M, K]
        bias = torch.randint(-9, 10, (N,), generator=g).float()
        aq, bq = O.cast_to_fp8(a, one, O.E4M3).cuda(), O.cast_to_fp8(b, one, O.E5M2).cuda()
        sa_inv, sb_inv = torch.tensor(3.0, device="cuda"), torch.tensor(0.75, device="cuda")
        prod = (b.double() @ a.double().t())
        want = (prod.float() * (sb_inv.cpu() * sa_inv.cpu()))
        e = torch.Tensor()
        ws = torch.empty(16, dtype=torch.int8, device="cuda")
        for od in (torch.float32, torch.bfloat16):
            D = torch.empty(M, N, dtype=od, device="cuda")
            tex.te_gemm(aq, sa_inv, tex.DType.kFloat8E4M3, True, bq, sb_inv, tex.DType.kFloat8E5M2, False,
                        D, e, tex.DType.kFloat32, e, bias.cuda(), tex.DType.kFloat32, e, False, ws, 16, False, True, 0)
            assert torch.equal(D.cpu(), (want + bias).to(od)), (M, N, K, od)
        D = torch.full((M, N), 7.0, device="cuda")
        tex.te_gemm(aq, sa_inv, tex.DType.kFloat8E4M3, True, bq, sb_inv, tex.DType.kFloat8E5M2, False,
                    D, e, tex.DType.kFloat32, e, torch.tensor([]), tex.DType.kFloat32, e, False, ws, 16, True, True, 0)
        assert torch.equal(D.cpu(), want + 7.0)
        # every transa / transb form, for every shape: operands read as they lie where the big kernel can, through
        # transposed copies elsewhere (small or ragged shapes, a bias, transa = transb = True)
        at = O.cast_to_fp8(a.t().contiguous(), one, O.E4M3).cuda()   # A as [K, N]
        bt = O.cast_to_fp8(b.t().contiguous(), one, O.E5M2).cuda()   # B as [K, M]
        for A_, ta, B_, tb in ((at, False, bq, False), (at, False, bt, True), (aq, True, bt, True)):
            D = torch.empty(M, N, device="cuda")
            tex.te_gemm(A_, sa_inv, tex.DType.kFloat8E4M3, ta, B_, sb_inv, tex.DType.kFloat8E5M2, tb,
                        D, e, tex.DType.kFloat32, e, torch.tensor([]), tex.DType.kFloat32, e, False, ws, 16, False, True, 0)
            assert torch.equal(D.cpu(), want), (M, N, K, ta, tb)
            D = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
            tex.te_gemm(A_, sa_inv, tex.DType.kFloat8E4M3, ta, B_, sb_inv, tex.DType.kFloat8E5M2, tb,
                        D, e, tex.DType.kFloat32, e, bias.cuda(), tex.DType.kFloat32, e, False, ws, 16, False, True, 0)
            assert torch.equal(D.cpu(), (want + bias).to(torch.bfloat16)), (M, N, K, ta, tb, "bias")
    with pytest.raises(RuntimeError):   # the bias-gradient epilogue is not served
        tex.te_gemm(aq, sa_inv, tex.DType.kFloat8E4M3, True, bq, sb_inv, tex.DType.kFloat8E5M2, False,
                    D, e, tex.DType.kFloat32, e, bias.cuda(), tex.DType.kFloat32, e, True, ws, 16, False, True, 0)


def test_te_gemm_fp8_output_with_scale_and_amax():
    tex = _tex()
    g = torch.Generator().manual_seed(6)
    one = torch.tensor(1.0)
    M, N, K = 512, 272, 256
    a = torch.randint(-4, 5, (N, K), generator=g).float()
    b = torch.randint(-4, 5, (M, K), generator=g).float()
    aq, bq = O.cast_to_fp8(a, one, O.E4M3).cuda(), O.cast_to_fp8(b, one, O.E4M3).cuda()
    r = (b.double() @ a.double().t()).float()
    d_scale = torch.tensor(0.5, device="cuda")
    for start in (0.0, 1e9):
        d_amax = torch.tensor(start, device="cuda")
        D = torch.empty(M, N, dtype=torch.uint8, device="cuda")
        e = torch.Tensor()
        tex.te_gemm(aq, one.cuda(), tex.DType.kFloat8E4M3, True, bq, one.cuda(), tex.DType.kFloat8E4M3, False,
                    D, d_scale, tex.DType.kFloat8E4M3, d_amax, torch.tensor([]), tex.DType.kFloat32, e, False,
                    torch.empty(1, dtype=torch.int8, device="cuda"), 1, False, False, 0)
        assert torch.equal(D.cpu(), O.cast_to_fp8(r, d_scale.cpu(), O.E4M3))
        assert d_amax.item() == max(start, r.abs().max().item())


def test_install_registers_the_names_the_reference_imports():
    import sys

    from nanotron_amd import tex_shim

    saved = {k: sys.modules.get(k) for k in ("transformer_engine", "transformer_engine_extensions")}
    try:
        tex_shim.install()
        import transformer_engine as te  # noqa: F401  (kernel.py:2)
        import transformer_engine_extensions as tex  # (kernel.py:3)

        assert tex is tex_shim and getattr(tex.DType, "kFloat32") == tex.DType.kFloat32
    finally:
        for k, v in saved.items():
            if v is None:
                sys.modules.pop(k, None)
            else:
                sys.modules[k] = v
