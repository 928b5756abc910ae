"""GPU parity of GEMMs whose B operand is given as its transpose, a [K, N] tensor (`ntfp8_gemm_desc.b_transposed`):
what the backward GEMMs of a linear layer have at hand where the reference calls tex.fp8_transpose first
(src/nanotron/fp8/kernel.py:43, src/nanotron/fp8/linear.py:104-109).  Integer-valued operands make every result
exact in any summation order, so the kernels are held to the fp64 product bit for bit; random operands must equal the
GEMM on the materialised transpose bit for bit (same tiles, same MFMA order)."""
import pytest
import torch

from oracle import fp8_oracle as O

pytestmark = pytest.mark.gpu


def _dt(fmt):
    from nanotron_amd.fp8 import DTypes

    return DTypes.FP8E4M3 if fmt == O.E4M3 else DTypes.FP8E5M2


def from_bytes(q_cpu, scale, fmt):
    from nanotron_amd.fp8 import FP8Tensor
    from nanotron_amd.fp8.meta import FP8Meta

    t = torch.Tensor._make_subclass(FP8Tensor, q_cpu.contiguous().cuda())
    t.fp8_meta = FP8Meta(torch.tensor(0.0, device="cuda"), torch.tensor(float(scale), dtype=torch.float32, device="cuda"),
                         _dt(fmt))
    return t


def _bits(t):
    return t.detach().float().cpu().contiguous().view(torch.int32)


def test_integer_operands_ragged_sweep_singly_and_batched():
    from nanotron_amd.fp8.kernel import _gemm_nt_batch

    rng = torch.Generator().manual_seed(31415)
    one = torch.tensor(1.0)
    shapes = [(2304, 2048, 400), (4096, 4352, 256), (129, 144, 256), (1000, 272, 1040)]   # half tiles only; whole + half; minimal
    for _ in range(10):
        shapes.append((int(torch.randint(129, 1400, (1,), generator=rng)), 16 * int(torch.randint(9, 88, (1,), generator=rng)),
                       16 * int(torch.randint(16, 130, (1,), generator=rng))))
    problems, wants = [], []
    for case, (M, N, K) in enumerate(shapes):
        fa, fb = [(O.E4M3, O.E4M3), (O.E5M2, O.E4M3), (O.E4M3, O.E5M2), (O.E5M2, O.E5M2)][case % 4]
        a = torch.randint(-4, 5, (M, K), generator=rng).float()
        bt = torch.randint(-4, 5, (K, N), generator=rng).float()
        A = from_bytes(O.cast_to_fp8(a, one, fa), 2.0, fa)
        Bt = from_bytes(O.cast_to_fp8(bt, one, fb), 0.5, fb)
        want = (a.double() @ bt.double()).float()   # scales 2 and 1/2 cancel
        assert torch.equal(want, O.gemm_nt(O.cast_to_fp8(a, one, fa), fa, torch.tensor(2.0), O.cast_to_fp8(bt.t().contiguous(), one, fb),
                                           fb, torch.tensor(0.5)))
        od = (torch.float32, torch.bfloat16, torch.float16)[case % 3]
        got = _gemm_nt_batch([(A, Bt, od, None, True)])[0]
        assert got.shape == (M, N) and got.dtype == od
        assert torch.equal(got.cpu(), want.to(od)), (M, N, K, fa, fb, od)
        if case % 3 == 0:   # fp32 accumulation into an existing buffer
            acc = torch.randint(-50, 50, (M, N), generator=rng).float()
            accg = acc.cuda()
            out = _gemm_nt_batch([(A, Bt, torch.float32, accg, True)])[0]
            assert out.data_ptr() == accg.data_ptr() and torch.equal(out.cpu(), want + acc)
        problems.append((A, Bt, od, None, True))
        wants.append(want.to(od))
    # one call: same formats share launches; a plain problem rides along in a launch of its own
    a = torch.randint(-4, 5, (300, 512), generator=rng).float()
    b = torch.randint(-4, 5, (272, 512), generator=rng).float()
    plain = (from_bytes(O.cast_to_fp8(a, one, O.E4M3), 1.0, O.E4M3), from_bytes(O.cast_to_fp8(b, one, O.E4M3), 1.0, O.E4M3),
             torch.float32, None)
    outs = _gemm_nt_batch(problems + [plain])
    for got, want in zip(outs, wants + [a @ b.t()]):
        assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("mnk", [(512, 768, 384), (2048, 4096, 4096), (4096, 1024, 1536), (1536, 1024, 4096)])
@pytest.mark.parametrize("fa,fb", [(O.E5M2, O.E4M3), (O.E4M3, O.E4M3)])
def test_random_operands_equal_the_gemm_on_the_materialised_transpose(mnk, fa, fb):
    from nanotron_amd.fp8 import FP8Tensor
    from nanotron_amd.fp8.kernel import _gemm_nt, _gemm_nt_batch

    M, N, K = mnk
    A = FP8Tensor(O.normal_tensor(M, (M, K), 1.0, torch.bfloat16).cuda(), _dt(fa))
    Bt = FP8Tensor(O.normal_tensor(N + 1, (K, N), 0.05, torch.bfloat16).cuda(), _dt(fb), with_transpose=True)
    for od in (torch.float32, torch.bfloat16):
        got = _gemm_nt_batch([(A, Bt, od, None, True)])[0]
        ref = _gemm_nt(A, Bt.transposed(), od, None)
        assert torch.equal(got, ref)
    # and against the oracle, at the GEMM tolerance
    r = O.gemm_nt(A.cpu().as_subclass(torch.Tensor), fa, A.fp8_meta.scale.cpu(),
                  Bt.transposed().cpu().as_subclass(torch.Tensor), fb, Bt.fp8_meta.scale.cpu())
    assert O.rel_l2(_gemm_nt_batch([(A, Bt, torch.float32, None, True)])[0].cpu(), r) <= 1e-3


def test_nan_and_inf_codes_travel_like_on_the_transposed_copy():
    from nanotron_amd.fp8.kernel import _gemm_nt, _gemm_nt_batch

    M, N, K = 300, 272, 384
    g = torch.Generator().manual_seed(9)
    one = torch.tensor(1.0)
    aq = O.cast_to_fp8(torch.randint(-4, 5, (M, K), generator=g).float(), one, O.E5M2)
    btq = O.cast_to_fp8(torch.randint(-4, 5, (K, N), generator=g).float(), one, O.E4M3)
    aq[7, 3] = 0x7C       # +Inf (e5m2)
    btq[100, 5] = 0x7F    # NaN (e4m3): column 5 of the result
    btq[383, 271] = 0xFF  # -NaN in the last row and column of B^T
    A, Bt = from_bytes(aq, 1.0, O.E5M2), from_bytes(btq, 1.0, O.E4M3)
    Bn = from_bytes(btq.t().contiguous(), 1.0, O.E4M3)
    got = _gemm_nt_batch([(A, Bt, torch.float32, None, True)])[0]
    ref = _gemm_nt(A, Bn, torch.float32, None)
    assert torch.isnan(got[:, 5]).all() and torch.isnan(got[:, 271]).all() and torch.isinf(got[7]).any()
    assert torch.equal(_bits(got), _bits(ref))


def test_requests_the_kernels_do_not_serve_are_refused():
    from nanotron_amd import _native as nt
    from nanotron_amd.fp8 import FP8Tensor
    from nanotron_amd.fp8.kernel import b_transposed_supported

    dev = torch.device("cuda", 0)
    unsupported = {nt.strerror(c): c for c in range(-8, 1)}["request not supported"]

    def call(M, N, K, d_dtype=nt.F32, scale_d=None):
        a = FP8Tensor(torch.randn(M, K, device=dev), _dt(O.E4M3))
        bt = FP8Tensor(torch.randn(K, N, device=dev), _dt(O.E4M3))
        out = torch.empty(M, N, dtype=torch.float32, device=dev)
        d = nt.GemmDesc()
        d.A, d.scale_a, d.B, d.scale_b, d.D = (a.data_ptr(), a.fp8_meta.scale.data_ptr(), bt.data_ptr(),
                                               bt.fp8_meta.scale.data_ptr(), out.data_ptr())
        d.M, d.N, d.K, d.fmt_a, d.fmt_b, d.d_dtype, d.accumulate, d.b_transposed = M, N, K, nt.E4M3, nt.E4M3, d_dtype, 0, 1
        if scale_d is not None:
            d.scale_d = scale_d.data_ptr()
        rc = nt.lib.ntfp8_gemm_batch((nt.GemmDesc * 1)(d), 1, nt.stream_ptr(dev))
        torch.cuda.synchronize()
        return rc

    assert call(256, 256, 256) == 0
    for M, N, K in [(256, 250, 256), (128, 256, 256), (256, 128, 256), (256, 256, 128), (256, 256, 250)]:
        assert not b_transposed_supported(M, N, K)
        assert call(M, N, K) == unsupported, (M, N, K)
    assert call(256, 256, 256, nt.OUT_E4M3, torch.ones(1, device=dev)) == 0              # fp8 outputs are served ...
    assert call(254, 256, 256, nt.OUT_E4M3, torch.ones(1, device=dev)) == unsupported    # ... for M a multiple of 4


@pytest.mark.parametrize("master", [torch.float32, torch.bfloat16])
def test_linear_gives_the_same_bits_with_and_without_transposed_copies(master):
    """FP8Linear over three delayed-scaling steps, once reading W and X as they are in the backward GEMMs, once on
    transposed copies: outputs, input gradients, weight gradients and scaling state agree bit for bit."""
    import nanotron_amd.fp8.kernel as K
    from nanotron_amd.fp8 import DTypes, FP8Linear, FP8Parameter

    T, H, I = 384, 512, 768
    w = O.normal_tensor(1, (I, H), 0.05, master)
    results = []
    for direct in (True, False):
        K.READ_B_TRANSPOSED = direct
        try:
            lin = FP8Linear(H, I, bias=False, device="cuda", dtype=master, out_dtype=torch.bfloat16, delayed_scaling=True,
                            amax_history_len=4, accumulate_grad=True)
            lin.weight = FP8Parameter(w.cuda(), DTypes.FP8E4M3)
            has_copy = getattr(lin.weight.data, "_transposed", None) is not None
            assert has_copy == (not direct)
            outs = []
            for step in range(3):
                x = O.normal_tensor(10 + step, (T, H), 1.0, torch.bfloat16).cuda().requires_grad_(True)
                gy = O.normal_tensor(20 + step, (T, I), 1e-2, torch.bfloat16).cuda()
                y = lin(x)
                y.backward(gy)
                lin.requantize_weight()
                grad = lin.weight.grad if master == torch.float32 else lin.weight.main_grad
                outs += [y.detach().clone(), x.grad.clone(), grad.clone()]
            outs += [st._buf.clone() for st in lin.scaling.values()]
            results.append(outs)
        finally:
            K.READ_B_TRANSPOSED = True
    for a, b in zip(*results):
        assert torch.equal(_bits(a), _bits(b))
    assert torch.isfinite(results[0][-4]).all() and results[0][-4].abs().max() > 0   # the accumulated weight gradient


def test_operator_falls_back_to_a_transposed_copy_when_the_direct_read_does_not_apply():
    """fp8_matmul_kernel(mat_a, transpose_a=False, ...) reads mat_a as it is where it can; a misaligned view, a shape
    with N not a multiple of 16, or a tensor that already carries its transposed copy take the copy.  Same results."""
    from nanotron_amd.fp8 import FP8Tensor
    from nanotron_amd.fp8.kernel import _operands, fp8_matmul_kernel
    from nanotron_amd.fp8.meta import FP8Meta

    one = torch.tensor(1.0)
    g = torch.Generator().manual_seed(4)
    K, N, M = 384, 272, 300
    w = torch.randint(-4, 5, (K, N), generator=g).float()     # mat_a [K, N]: reduced over its rows
    x = torch.randint(-4, 5, (M, K), generator=g).float()     # mat_b [M, K]
    want = x @ w
    X = from_bytes(O.cast_to_fp8(x, one, O.E4M3), 1.0, O.E4M3)
    W = from_bytes(O.cast_to_fp8(w, one, O.E4M3), 1.0, O.E4M3)
    assert _operands(W, False, X, False)[2] is True
    assert torch.equal(fp8_matmul_kernel(W, False, X, False, False).cpu(), want)
    # misaligned storage
    buf = torch.empty(K * N + 8, dtype=torch.uint8, device="cuda")
    view = buf[8:].view(K, N)
    view.copy_(W.as_subclass(torch.Tensor))
    Wm = torch.Tensor._make_subclass(FP8Tensor, view)
    Wm.fp8_meta = FP8Meta(torch.tensor(0.0, device="cuda"), torch.tensor(1.0, device="cuda"), _dt(O.E4M3))
    assert Wm.data_ptr() % 16 == 8 and _operands(Wm, False, X, False)[2] is False
    assert torch.equal(fp8_matmul_kernel(Wm, False, X, False, False).cpu(), want)
    # a tensor that carries its transposed copy uses it
    W2 = from_bytes(O.cast_to_fp8(w, one, O.E4M3), 1.0, O.E4M3)
    W2.transposed()
    assert _operands(W2, False, X, False)[2] is False
    assert torch.equal(fp8_matmul_kernel(W2, False, X, False, False).cpu(), want)
    # N not a multiple of 16
    w3 = torch.randint(-4, 5, (K, 250), generator=g).float()
    W3 = from_bytes(O.cast_to_fp8(w3, one, O.E4M3), 1.0, O.E4M3)
    assert _operands(W3, False, X, False)[2] is False
    assert torch.equal(fp8_matmul_kernel(W3, False, X, False, False).cpu(), x @ w3)


# ------------------------------------------------------------------------------------------ both operands transposed
def test_a_and_b_transposed_integer_sweep_singly_and_batched():
    """The wgrad form: D[M,N] = A^T . B with A given as [K, M] and B as [K, N] (`a_transposed` next to `b_transposed`).
    Integer operands: exact in any order, so whole tiles, half tiles, ragged edges, K tails, every format pair and
    output type must equal the fp64 product; then all of them in one call next to plain and B-transposed problems."""
    from nanotron_amd.fp8.kernel import _gemm_nt_batch

    rng = torch.Generator().manual_seed(271828)
    one = torch.tensor(1.0)
    shapes = [(2304, 2048, 400), (4096, 4352, 256), (144, 144, 256), (1008, 272, 1040), (6144, 4096, 512)]
    for _ in range(9):
        shapes.append((16 * int(torch.randint(9, 88, (1,), generator=rng)), 16 * int(torch.randint(9, 88, (1,), generator=rng)),
                       16 * int(torch.randint(16, 130, (1,), generator=rng))))
    problems, wants = [], []
    for case, (M, N, K) in enumerate(shapes):
        fa, fb = [(O.E5M2, O.E4M3), (O.E4M3, O.E4M3), (O.E4M3, O.E5M2), (O.E5M2, O.E5M2)][case % 4]
        at = torch.randint(-4, 5, (K, M), generator=rng).float()
        bt = torch.randint(-4, 5, (K, N), generator=rng).float()
        At = from_bytes(O.cast_to_fp8(at, one, fa), 0.5, fa)
        Bt = from_bytes(O.cast_to_fp8(bt, one, fb), 2.0, fb)
        want = (at.double().t() @ bt.double()).float()
        od = (torch.float32, torch.bfloat16, torch.float16)[case % 3]
        got = _gemm_nt_batch([(At, Bt, od, None, True, None, True)])[0]
        assert got.shape == (M, N) and got.dtype == od
        assert torch.equal(got.cpu(), want.to(od)), (M, N, K, fa, fb, od)
        if case % 3 == 0:
            acc = torch.randint(-50, 50, (M, N), generator=rng).float()
            accg = acc.cuda()
            out = _gemm_nt_batch([(At, Bt, torch.float32, accg, True, None, True)])[0]
            assert out.data_ptr() == accg.data_ptr() and torch.equal(out.cpu(), want + acc)
        problems.append((At, Bt, od, None, True, None, True))
        wants.append(want.to(od))
    # a dgrad-shaped problem (A plain, B transposed) and a plain one ride along: operand layout is per problem
    a = torch.randint(-4, 5, (640, 512), generator=rng).float()
    b_t = torch.randint(-4, 5, (512, 272), generator=rng).float()
    b = torch.randint(-4, 5, (272, 512), generator=rng).float()
    A = from_bytes(O.cast_to_fp8(a, one, O.E5M2), 1.0, O.E5M2)
    problems.append((A, from_bytes(O.cast_to_fp8(b_t, one, O.E4M3), 1.0, O.E4M3), torch.float32, None, True))
    wants.append(a @ b_t)
    problems.append((A, from_bytes(O.cast_to_fp8(b, one, O.E4M3), 1.0, O.E4M3), torch.float32, None))
    wants.append(a @ b.t())
    for got, want in zip(_gemm_nt_batch(problems), wants):
        assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("mnk", [(768, 512, 384), (4096, 4096, 2048), (1536, 1024, 4096), (6144, 4096, 4096)])
def test_a_transposed_random_operands_equal_the_gemm_on_materialised_transposes(mnk):
    """Same tiles, same MFMA order: reading dY and X as they are must give the bits of the GEMM on their transposed
    copies, whole tiles and half-tile tail alike; and the oracle's result within the GEMM tolerance."""
    from nanotron_amd.fp8 import FP8Tensor
    from nanotron_amd.fp8.kernel import _gemm_nt, _gemm_nt_batch

    M, N, K = mnk
    At = FP8Tensor(O.normal_tensor(M, (K, M), 1e-2, torch.bfloat16).cuda(), _dt(O.E5M2), with_transpose=True)
    Bt = FP8Tensor(O.normal_tensor(N + 1, (K, N), 1.0, torch.bfloat16).cuda(), _dt(O.E4M3), with_transpose=True)
    for od in (torch.float32, torch.bfloat16):
        got = _gemm_nt_batch([(At, Bt, od, None, True, None, True)])[0]
        ref = _gemm_nt(At.transposed(), Bt.transposed(), od, None)
        assert torch.equal(got, ref)
    r = O.gemm_nt(At.transposed().cpu().as_subclass(torch.Tensor), O.E5M2, At.fp8_meta.scale.cpu(),
                  Bt.transposed().cpu().as_subclass(torch.Tensor), O.E4M3, Bt.fp8_meta.scale.cpu())
    assert O.rel_l2(_gemm_nt_batch([(At, Bt, torch.float32, None, True, None, True)])[0].cpu(), r) <= 1e-3


def test_a_transposed_requests_the_kernels_do_not_serve_are_refused():
    from nanotron_amd import _native as nt
    from nanotron_amd.fp8 import FP8Tensor
    from nanotron_amd.fp8.kernel import a_transposed_supported

    dev = torch.device("cuda", 0)

    def call(M, N, K, bt=1):
        a = FP8Tensor(torch.randn(K, M, device=dev), _dt(O.E4M3))
        b = FP8Tensor(torch.randn(K, N, device=dev), _dt(O.E4M3))
        out = torch.empty(M, N, dtype=torch.float32, device=dev)
        d = nt.GemmDesc()
        d.A, d.scale_a, d.B, d.scale_b, d.D = a.data_ptr(), a.fp8_meta.scale.data_ptr(), b.data_ptr(), b.fp8_meta.scale.data_ptr(), out.data_ptr()
        d.M, d.N, d.K, d.fmt_a, d.fmt_b, d.d_dtype, d.b_transposed, d.a_transposed = M, N, K, nt.E4M3, nt.E4M3, nt.F32, bt, 1
        rc = nt.lib.ntfp8_gemm_batch((nt.GemmDesc * 1)(d), 1, nt.stream_ptr(dev))
        torch.cuda.synchronize()
        return rc

    assert a_transposed_supported(256, 256, 256) and call(256, 256, 256) == 0
    assert call(256, 256, 256, bt=0) == -5                       # only next to a transposed B
    for M, N, K in [(250, 256, 256), (256, 250, 256), (128, 256, 256), (256, 256, 128)]:
        assert not a_transposed_supported(M, N, K)
        assert call(M, N, K) == -5, (M, N, K)


def test_linear_backward_reads_the_output_gradient_as_it_is():
    """FP8Linear's wgrad takes dY without a transposed copy when the shape allows it, and gives the bits of the path on
    transposed copies."""
    import nanotron_amd.fp8.kernel as K
    from nanotron_amd.fp8 import DTypes, FP8Linear, FP8Parameter, FP8Tensor

    T, H, I = 384, 512, 768
    w = O.normal_tensor(1, (I, H), 0.05, torch.bfloat16)
    seen, results = [], []
    orig = FP8Tensor.__new__

    def spy(cls, tensor, dtype, **kw):
        if dtype == DTypes.FP8E5M2:
            seen.append(bool(kw.get("with_transpose")))
        return orig(cls, tensor, dtype, **kw)

    for direct in (True, False):
        K.READ_A_TRANSPOSED = direct
        FP8Tensor.__new__ = spy
        try:
            lin = FP8Linear(H, I, bias=False, device="cuda", dtype=torch.bfloat16, out_dtype=torch.bfloat16, delayed_scaling=True)
            lin.weight = FP8Parameter(w.cuda(), DTypes.FP8E4M3)
            outs = []
            for step in range(3):
                x = O.normal_tensor(10 + step, (T, H), 1.0, torch.bfloat16).cuda().requires_grad_(True)
                lin(x).backward(O.normal_tensor(20 + step, (T, I), 1e-2, torch.bfloat16).cuda())
                outs += [x.grad.clone(), lin.weight.main_grad.clone()]
            results.append(outs)
        finally:
            K.READ_A_TRANSPOSED = True
            FP8Tensor.__new__ = orig
    assert seen == [False] * 3 + [True] * 3
    for a, b in zip(*results):
        assert torch.equal(_bits(a), _bits(b))
