"""GPU parity of the FP8 GEMM (C ABI ntfp8_gemm / fp8_matmul_kernel) against the CPU oracle:
bit-exact where the arithmetic is exact in any order, rel-L2 <= 1e-3 otherwise."""
import pytest
import torch

from oracle import fp8_oracle as O

pytestmark = pytest.mark.gpu

REL_L2 = 1e-3  # tolerance stated for the GEMMs: rel-L2 against fp32 matmul of exactly-upcast operands
FMTS = [O.E4M3, O.E5M2]


def _dt(fmt):
    from nanotron_amd.fp8 import DTypes

    return DTypes.FP8E4M3 if fmt == O.E4M3 else DTypes.FP8E5M2


def gpu_quant(x, fmt, with_transpose=False):
    from nanotron_amd.fp8 import FP8Tensor

    return FP8Tensor(x.cuda(), _dt(fmt), with_transpose=with_transpose)


def gpu_gemm_nt(aq, bq, out_dtype=torch.float32, accumulate_into=None):
    from nanotron_amd.fp8.kernel import _gemm_nt

    return _gemm_nt(aq, bq, out_dtype, accumulate_into)


def from_bytes(q_cpu, scale, fmt):
    """FP8Tensor on the GPU from given bytes + scale (no quantisation involved)."""
    from nanotron_amd.fp8 import FP8Tensor
    from nanotron_amd.fp8.meta import FP8Meta

    t = torch.Tensor._make_subclass(FP8Tensor, q_cpu.cuda())
    t.fp8_meta = FP8Meta(torch.tensor(0.0, device="cuda"), torch.tensor(float(scale), dtype=torch.float32, device="cuda"),
                         _dt(fmt))
    return t


@pytest.mark.parametrize("fa", FMTS)
@pytest.mark.parametrize("fb", FMTS)
@pytest.mark.parametrize("mnk", [(33, 17, 96), (128, 128, 128), (130, 250, 272), (64, 64, 16), (5, 3, 7), (16, 16, 16),
                                 (1, 1, 1), (200, 36, 1040)])
def test_integer_operands_bit_exact(fa, fb, mnk):
    M, N, K = mnk
    g = torch.Generator().manual_seed(M * 7 + N * 3 + K)
    a = torch.randint(-8, 9, (M, K), generator=g).float()
    b = torch.randint(-8, 9, (N, K), generator=g).float()
    one = torch.tensor(1.0)
    aq, bq = O.cast_to_fp8(a, one, fa), O.cast_to_fp8(b, one, fb)
    want = O.gemm_nt(aq, fa, one, bq, fb, one)
    assert torch.equal(want, (a.double() @ b.double().t()).float())
    A, B = from_bytes(aq, 1.0, fa), from_bytes(bq, 1.0, fb)
    got = gpu_gemm_nt(A, B).cpu()
    assert torch.equal(got, want)
    for od in (torch.bfloat16, torch.float16):
        assert torch.equal(gpu_gemm_nt(A, B, od).cpu(), want.to(od))
    acc = torch.randint(-100, 100, (M, N), generator=g).float()
    accg = acc.cuda()
    out = gpu_gemm_nt(A, B, torch.float32, accg)
    assert out.data_ptr() == accg.data_ptr() and torch.equal(out.cpu(), want + acc)
    # power-of-two scales: the descale is exact too
    A2, B2 = from_bytes(aq, 4.0, fa), from_bytes(bq, 0.5, fb)
    assert torch.equal(gpu_gemm_nt(A2, B2).cpu(), want * 0.5)


@pytest.mark.parametrize("mnk,fa,fb", [
    ((4096, 4096, 272), O.E4M3, O.E4M3),    # 256 whole 256x256 tiles (one per CU), K tail of 16
    ((4096, 6144, 256), O.E5M2, O.E4M3),    # 384 tiles: one whole round + 128 tiles as 128-row halves; two K-tiles
    ((4000, 4136, 400), O.E4M3, O.E5M2),    # 272 tiles with ragged bottom / right edges, odd K-tile count
    ((2304, 2048, 1024), O.E4M3, O.E4M3),   # 72 tiles: every tile computed as halves
])
def test_large_grid_bit_exact(mnk, fa, fb):
    """Shapes with enough tiles for the whole-tile kernel (the small shapes above only reach the
    half-tile one); small integers keep every partial sum exact, so any order must give these bits."""
    M, N, K = mnk
    g = torch.Generator().manual_seed(M + 3 * N + 5 * K)
    a = torch.randint(-4, 5, (M, K), generator=g).float()
    b = torch.randint(-4, 5, (N, K), generator=g).float()
    one = torch.tensor(1.0)
    aq, bq = O.cast_to_fp8(a, one, fa), O.cast_to_fp8(b, one, fb)
    want = (a @ b.t())  # |sum| <= 16 K < 2^24: exact in fp32 in any order
    A, B = from_bytes(aq, 1.0, fa), from_bytes(bq, 1.0, fb)
    assert torch.equal(gpu_gemm_nt(A, B).cpu(), want)
    for od in (torch.bfloat16, torch.float16):
        assert torch.equal(gpu_gemm_nt(A, B, od).cpu(), want.to(od))
    acc = torch.randint(-100, 100, (M, N), generator=g).float()
    accg = acc.cuda()
    assert torch.equal(gpu_gemm_nt(A, B, torch.float32, accg).cpu(), want + acc)
    A2, B2 = from_bytes(aq, 0.25, fa), from_bytes(bq, 8.0, fb)
    assert torch.equal(gpu_gemm_nt(A2, B2, torch.bfloat16).cpu(), (want * 0.5).to(torch.bfloat16))


def test_every_fp8_code_decodes_like_the_oracle():
    # A = one row per code (one-hot in K), B = identity-like selectors: D[i, j] = decode(code i) * [i == j]
    for fmt in FMTS:
        codes = torch.arange(256, dtype=torch.uint8)
        vals = O.upcast(codes, fmt)
        keep = torch.isfinite(vals)
        a = torch.zeros(256, 256, dtype=torch.uint8)
        a[torch.arange(256), torch.arange(256)] = torch.where(keep, codes, torch.zeros_like(codes))
        eye = O.cast_to_fp8(torch.eye(256), torch.tensor(1.0), O.E4M3)
        got = gpu_gemm_nt(from_bytes(a, 1.0, fmt), from_bytes(eye, 1.0, O.E4M3)).cpu()
        want = torch.diag(torch.where(keep, vals, torch.zeros_like(vals)))
        assert torch.equal(got, want)


@pytest.mark.parametrize("fa,fb", [(O.E4M3, O.E4M3), (O.E5M2, O.E4M3)])
@pytest.mark.parametrize("mnk", [(256, 256, 512), (300, 200, 1024), (64, 1000, 144), (129, 127, 2048), (96, 80, 100)])
@pytest.mark.parametrize("od", [torch.float32, torch.bfloat16])
def test_random_operands_rel_l2(fa, fb, mnk, od):
    M, N, K = mnk
    a = O.quantise_current(O.normal_tensor(M + K, (M, K), 1.0 if fa == O.E4M3 else 1e-3), fa)
    b = O.quantise_current(O.normal_tensor(N + K + 1, (N, K), 0.02), fb)
    ref32 = O.gemm_nt(a.q, fa, a.scale, b.q, fb, b.scale, od)
    ref64 = O.gemm_nt(a.q, fa, a.scale, b.q, fb, b.scale, torch.float64, None, torch.float64)
    got = gpu_gemm_nt(from_bytes(a.q, a.scale, fa), from_bytes(b.q, b.scale, fb), od).cpu()
    assert got.dtype == od
    tol = REL_L2 if od == torch.float32 else 4e-3  # bf16 output rounding alone is ~2e-3 rel-L2
    assert O.rel_l2(got, ref32) <= REL_L2
    assert O.rel_l2(got, ref64) <= tol
    if od == torch.float32:
        # the matrix cores align and truncate products inside one 64-deep dot product, so the error
        # sits a little above a pure fp32 FMA chain (measured ~1.5e-5): far inside the 1e-3 gate
        assert O.rel_l2(got, ref64) <= 1e-4


def test_fp8_matmul_kernel_operator_meaning_all_flag_combinations():
    from nanotron_amd.fp8.kernel import fp8_matmul_kernel

    X = O.quantise_current(O.normal_tensor(31, (48, 32), 1.0), O.E4M3)
    W = O.quantise_current(O.normal_tensor(32, (80, 32), 0.02), O.E4M3)
    G = O.quantise_current(O.normal_tensor(33, (48, 80), 1e-3), O.E5M2)
    Xg, Wg, Gg = (from_bytes(t.q, t.scale, t.fmt) for t in (X, W, G))
    cases = [
        (Wg, True, Xg, False, W, X),    # forward  X.W^T            (linear.py:82-84)
        (Wg, False, Gg, False, W, G),   # dgrad    dY.W
        (Xg, False, Gg, True, X, G),    # wgrad    dY^T.X
        (Gg, True, Xg, True, G, X),     # X^T.dY^T = (dY.X)^T shape [32,48] needs K match: G[48,80]^T.. skipped below
    ]
    for i, (a, ta, b, tb, ao, bo) in enumerate(cases[:3]):
        got = fp8_matmul_kernel(a, ta, b, tb, use_split_accumulator=bool(i)).cpu()
        want = O.fp8_matmul_kernel(ao.q, ao.fmt, ao.scale, ta, bo.q, bo.fmt, bo.scale, tb)
        assert got.shape == want.shape and got.dtype == torch.float32
        assert O.rel_l2(got, want) <= 1e-4
    # both transposed: D = B^T . A^T with A [48,32], B [80,48]  ->  [80... ] use compatible shapes
    A = O.quantise_current(O.normal_tensor(41, (40, 24), 1.0), O.E4M3)
    B = O.quantise_current(O.normal_tensor(42, (24, 56), 1.0), O.E4M3)
    got = fp8_matmul_kernel(from_bytes(A.q, A.scale, A.fmt), True, from_bytes(B.q, B.scale, B.fmt), True, False).cpu()
    want = O.fp8_matmul_kernel(A.q, A.fmt, A.scale, True, B.q, B.fmt, B.scale, True)
    assert got.shape == (56, 40) and O.rel_l2(got, want) <= 1e-4


def test_config1_single_linear_forward():
    """Benchmark config 1: X bf16 [2048,1024] ~N(0,1), W bf16 [1024,1024] ~N(0,0.02), both e4m3,
    delayed scaling (history 16, margin 0; first step = current scaling), bf16 output."""
    from nanotron_amd.fp8 import DelayedScaling, DTypes, FP8Tensor

    x = O.normal_tensor(1234 + 100, (2048, 1024), 1.0)
    w = O.normal_tensor(1234 + 101, (1024, 1024), 0.02)
    sx, sw = DelayedScaling(DTypes.FP8E4M3), DelayedScaling(DTypes.FP8E4M3)
    rx, rw = O.DelayedScaling(O.E4M3), O.DelayedScaling(O.E4M3)
    xq, wq = rx.quantise(x), rw.quantise(w)
    xg = FP8Tensor(x.cuda(), DTypes.FP8E4M3, state=sx)
    wg = FP8Tensor(w.cuda(), DTypes.FP8E4M3, state=sw)
    assert torch.equal(xg.cpu().as_subclass(torch.Tensor), xq.q) and torch.equal(wg.cpu().as_subclass(torch.Tensor), wq.q)
    assert xg.fp8_meta.scale.item() == xq.scale.item() and wg.fp8_meta.scale.item() == wq.scale.item()
    got = gpu_gemm_nt(xg, wg, torch.bfloat16).cpu()
    ref = O.linear_forward(xq, wq, torch.float32)
    assert O.rel_l2(gpu_gemm_nt(xg, wg, torch.float32).cpu(), ref) <= REL_L2
    assert torch.equal(got, gpu_gemm_nt(xg, wg, torch.float32).cpu().to(torch.bfloat16))


def _sampled_rows_check(aq, bq, got, rows, acc=None, tol=REL_L2):
    ref = O.gemm_nt(aq.q[rows], aq.fmt, aq.scale, bq.q, bq.fmt, bq.scale)
    if acc is not None:
        ref = ref + acc[rows]
    assert O.rel_l2(got[rows].float(), ref) <= tol


def test_config3_and_4_llama7b_mlp_shapes():
    """Benchmark configs 3 and 4: M=4096, hidden 4096, intermediate 11008; forward GEMMs with bf16
    output, dgrad with bf16 output, wgrad accumulated into a pre-filled fp32 buffer.  Checked on
    sampled output rows (the oracle on all rows would take minutes)."""
    M, H, I = 4096, 4096, 11008
    x = gpu_quant(O.normal_tensor(1534, (M, H), 1.0), O.E4M3, with_transpose=True)
    wu = gpu_quant(O.normal_tensor(1535, (I, H), 0.02), O.E4M3, with_transpose=True)
    wd = gpu_quant(O.normal_tensor(1536, (H, I), 0.02), O.E4M3, with_transpose=True)
    h = gpu_quant(O.normal_tensor(1537, (M, I), 1.0), O.E4M3, with_transpose=True)
    gy = gpu_quant(O.normal_tensor(1634, (M, I), 1e-3), O.E5M2, with_transpose=True)
    gd = gpu_quant(O.normal_tensor(1635, (M, H), 1e-3), O.E5M2, with_transpose=True)

    def cpu(t, fmt):
        return O.Quantised(t.cpu().as_subclass(torch.Tensor), t.fp8_meta.amax.cpu(), t.fp8_meta.scale.cpu(), fmt)

    rows = torch.tensor([0, 1, 127, 128, 2047, 4095])
    # forward up/gate [M,I] and down [M,H]
    y = gpu_gemm_nt(x, wu, torch.bfloat16).cpu()
    _sampled_rows_check(cpu(x, O.E4M3), cpu(wu, O.E4M3), y, rows, tol=4e-3)
    y = gpu_gemm_nt(h, wd, torch.bfloat16).cpu()
    _sampled_rows_check(cpu(h, O.E4M3), cpu(wd, O.E4M3), y, rows, tol=4e-3)
    # dgrad: dX[M,H] = dY[M,I] . Wu[I,H]  ->  gemm_nt(dY, Wu^T)
    dx = gpu_gemm_nt(gy, wu.transposed(), torch.float32).cpu()
    _sampled_rows_check(cpu(gy, O.E5M2), cpu(wu.transposed(), O.E4M3), dx, rows)
    # wgrad: dWu[I,H] = dY^T[I,M] . X[M,H]  ->  gemm_nt(dY^T, X^T), accumulated into fp32 master grads
    acc = O.normal_tensor(99, (I, H), 1.0, torch.float32)
    accg = acc.cuda()
    gpu_gemm_nt(gy.transposed(), x.transposed(), torch.float32, accg)
    rows_w = torch.tensor([0, 5, 4096, 11007])
    _sampled_rows_check(cpu(gy.transposed(), O.E5M2), cpu(x.transposed(), O.E4M3), accg.cpu(), rows_w, acc=acc)
    # dWd[H,I] = gd^T[H,M] . h[M,I]
    dwd = gpu_gemm_nt(gd.transposed(), h.transposed(), torch.float32).cpu()
    _sampled_rows_check(cpu(gd.transposed(), O.E5M2), cpu(h.transposed(), O.E4M3), dwd, torch.tensor([0, 77, 4095]))


def test_batched_gemms_equal_separate_calls():
    """ntfp8_gemm_batch: problems of one format pair share launches (their tiles form one list, longest K first),
    others go out on their own; whatever the grouping, every output must equal the separate call bit for bit."""
    from nanotron_amd.fp8.kernel import _gemm_nt_batch

    def q(seed, shape, fmt, std=1.0):
        return gpu_quant(O.normal_tensor(seed, shape, std), fmt, with_transpose=True)

    x = q(1, (4096, 1024), O.E4M3)        # activations [M, K]
    w = q(2, (1536, 1024), O.E4M3, 0.02)  # weight [N, K]
    g = q(3, (4096, 1536), O.E5M2, 1e-3)  # output gradient [M, N]
    small_a, small_b = q(4, (96, 160), O.E4M3), q(5, (80, 160), O.E4M3)
    acc0 = O.normal_tensor(6, (1536, 1024), 1.0, torch.float32)
    problems = [
        (g, w.transposed(), torch.bfloat16, None),                  # dgrad  4096x1024x1536, e5m2 x e4m3
        (g.transposed(), x.transposed(), torch.float32, None),      # wgrad  1536x1024x4096, e5m2 x e4m3, fp32
        (x, w, torch.bfloat16, None),                               # fwd    4096x1536x1024, e4m3 x e4m3
        (small_a, small_b, torch.float16, None),                    # served by the small kernel
        (g.transposed(), x.transposed(), torch.float32, acc0.cuda()),  # wgrad accumulated into a master buffer
        (g, w.transposed(), torch.float32, None),                   # a fifth e5m2 x e4m3 problem (> 4 per launch)
        (g, w.transposed(), torch.float16, None),
    ]
    want = []
    for a, b, dt, acc in problems:
        want.append(gpu_gemm_nt(a, b, dt, None if acc is None else acc0.cuda()).cpu())
    got = _gemm_nt_batch(problems)
    assert len(got) == len(problems)
    for (a, b, dt, acc), o, w_ in zip(problems, got, want):
        assert o.dtype == (torch.float32 if acc is not None else dt)
        if acc is not None:
            assert o.data_ptr() == acc.data_ptr()
        assert torch.equal(o.cpu(), w_)
    # and against the oracle for the pair a backward issues
    cpu = lambda t, fmt: O.Quantised(t.cpu().as_subclass(torch.Tensor), t.fp8_meta.amax.cpu(), t.fp8_meta.scale.cpu(), fmt)
    dx = O.linear_dgrad(cpu(g, O.E5M2), cpu(w, O.E4M3), torch.bfloat16)
    dw = O.linear_wgrad(cpu(g, O.E5M2), cpu(x, O.E4M3))
    assert O.rel_l2(got[0].float().cpu(), dx.float()) <= 4e-3
    assert O.rel_l2(got[1].cpu(), dw) <= REL_L2


def test_batched_gemm_rejects_dependent_problems():
    from nanotron_amd import _native as nt
    from nanotron_amd.fp8.kernel import _gemm_nt_batch

    a = gpu_quant(O.normal_tensor(11, (256, 256), 1.0), O.E4M3)
    b = gpu_quant(O.normal_tensor(12, (256, 256), 1.0), O.E4M3)
    out = torch.empty(256, 256, dtype=torch.float32, device="cuda")
    with pytest.raises(RuntimeError):  # both problems write the same output
        _gemm_nt_batch([(a, b, torch.float32, out), (b, a, torch.float32, out)])
    descs = (nt.GemmDesc * 1)()
    assert nt.lib.ntfp8_gemm_batch(descs, 0, None) == -3   # NTFP8_ERR_SIZE
    assert nt.lib.ntfp8_gemm_batch(descs, 1, None) == -1   # NTFP8_ERR_NULL: empty descriptor
    assert nt.lib.ntfp8_gemm_batch(None, 1, None) == -1


def test_ragged_shapes_bit_exact_sweep():
    """Seeded sweep over ragged shapes that take the large-tile kernels (edges in M and N, K tails of every
    multiple of 16, odd and even K-tile counts, whole and half tiles), singly and as one batch."""
    from nanotron_amd.fp8.kernel import _gemm_nt_batch

    rng = torch.Generator().manual_seed(2718)
    one = torch.tensor(1.0)
    problems, wants = [], []
    for case in range(14):
        M = int(torch.randint(129, 1400, (1,), generator=rng))
        N = int(torch.randint(129, 1400, (1,), generator=rng))
        K = 16 * int(torch.randint(16, 130, (1,), generator=rng))
        fa, fb = (O.E5M2, O.E4M3) if case % 3 else (O.E4M3, O.E4M3)
        a = torch.randint(-4, 5, (M, K), generator=rng).float()
        b = torch.randint(-4, 5, (N, K), generator=rng).float()
        A, B = from_bytes(O.cast_to_fp8(a, one, fa), 1.0, fa), from_bytes(O.cast_to_fp8(b, one, fb), 1.0, fb)
        want = a @ b.t()
        od = (torch.float32, torch.bfloat16, torch.float16)[case % 3]
        assert torch.equal(gpu_gemm_nt(A, B, od).cpu(), want.to(od)), (M, N, K, od)
        problems.append((A, B, od, None))
        wants.append(want.to(od))
    for got, want in zip(_gemm_nt_batch(problems), wants):
        assert torch.equal(got.cpu(), want)
