from typing import Optional, Union

import torch

from nanotron_amd import _native as nt
from nanotron_amd.fp8.dtypes import DTypes
from nanotron_amd.fp8.tensor import DelayedScaling, FP8Tensor

_FMT = {DTypes.FP8E4M3: nt.E4M3, DTypes.FP8E5M2: nt.E5M2}
_OUT_FMT = {DTypes.FP8E4M3: nt.OUT_E4M3, DTypes.FP8E5M2: nt.OUT_E5M2}


def _bytes_and_meta(t: FP8Tensor):
    """(contiguous uint8 tensor, meta) of an fp8 operand.  The meta is a Python attribute of the FP8Tensor object: a
    copy made by `.contiguous()` (of a view such as a slice or `.t()`) does not carry it, so it is read first."""
    meta = t.fp8_meta
    raw = t.as_subclass(torch.Tensor)
    return (raw if raw.is_contiguous() else raw.contiguous()), meta


def _check_bias(bias: torch.Tensor, N: int, dev) -> torch.Tensor:
    assert bias.dim() == 1 and bias.shape[0] == N and bias.device == dev, (tuple(bias.shape), N)
    assert bias.dtype in nt.TORCH_TO_NT, f"unsupported bias dtype {bias.dtype}"
    return bias.detach().contiguous()


def _gemm_nt(a: FP8Tensor, b: FP8Tensor, out_dtype: torch.dtype, accumulate_into: Optional[torch.Tensor],
             bias: Optional[torch.Tensor] = None):
    """D[M,N] = A[M,K] . B[N,K]^T, descaled (te_gemm's TN form, src/nanotron/fp8/kernel.py:46-68); with `bias`
    [N] added to the descaled fp32 result before the single rounding (te_gemm's bias argument, which the
    reference leaves empty, kernel.py:29-32)."""
    if bias is not None:
        return _gemm_nt_batch([(a, b, out_dtype, accumulate_into, False, bias)])[0]
    assert a.dim() == 2 and b.dim() == 2 and a.shape[1] == b.shape[1], (tuple(a.shape), tuple(b.shape))
    M, K = a.shape
    N = b.shape[0]
    dev = a.device
    a, ma = _bytes_and_meta(a)
    b, mb = _bytes_and_meta(b)
    if accumulate_into is not None:
        assert accumulate_into.dtype == torch.float32 and accumulate_into.shape == (M, N)
        assert accumulate_into.is_contiguous() and accumulate_into.device == dev
        out, acc = accumulate_into, 1
    else:
        out, acc = torch.empty((M, N), dtype=out_dtype, device=dev), 0
    nt.check(nt.lib.ntfp8_gemm(a.data_ptr(), _FMT[ma.dtype], ma.scale.data_ptr(),
                               b.data_ptr(), _FMT[mb.dtype], mb.scale.data_ptr(),
                               out.data_ptr(), nt.TORCH_TO_NT[out.dtype], M, N, K, acc, nt.stream_ptr(dev)),
             "ntfp8_gemm")
    return out


def _gemm_nt_fp8(a: FP8Tensor, b: FP8Tensor, dtype: DTypes, state: Optional[DelayedScaling],
                 with_transpose: bool, bias: Optional[torch.Tensor] = None, bt: bool = False, at: bool = False) -> FP8Tensor:
    """FP8Tensor(_gemm_nt(a, b, float32), dtype, state=state, with_transpose=with_transpose), bit for bit, with the
    fp32 result never written to memory: the GEMM epilogue casts with the scale `state` holds from earlier steps,
    leaves max|result| behind, and a one-wave kernel turns that into amax, history roll and next scale.

    The amax of a GEMM result is not known before the GEMM has run, so a step without a held scale (no `state`, or
    one that has not seen a usable amax yet) goes the long way: fp32 result, then the ordinary quantisation."""
    from nanotron_amd.fp8.meta import FP8Meta

    assert dtype in _OUT_FMT, f"{dtype} is not an FP8 format"
    if state is None or not state.known_initialised:
        hp = (_gemm_nt_batch([(a, b, torch.float32, None, True, None, at)])[0] if bt
              else _gemm_nt(a, b, torch.float32, None, bias))
        return FP8Tensor(hp, dtype, state=state, with_transpose=with_transpose)
    assert state.dtype == dtype, "delayed-scaling state was created for another format"
    assert a.dim() == 2 and b.dim() == 2 and a.shape[0 if at else 1] == b.shape[0 if bt else 1], \
        (tuple(a.shape), tuple(b.shape), bt, at)
    assert not at or bt, "a transposed A operand is only read next to a transposed B operand"
    assert bias is None or not bt, "no bias together with a transposed B operand"
    K, M = a.shape if at else a.shape[::-1]
    N = b.shape[1 if bt else 0]
    dev = a.device
    assert state._buf.device == dev
    a, ma = _bytes_and_meta(a)
    b, mb = _bytes_and_meta(b)
    if bias is not None:
        bias = _check_bias(bias, N, dev)
    out = torch.empty((M, N), dtype=torch.uint8, device=dev)
    out_t = torch.empty((N, M), dtype=torch.uint8, device=dev) if with_transpose else None
    scalars = torch.empty(2, dtype=torch.float32, device=dev)  # [amax, scale used]
    ws, st = nt.workspace_and_stream(dev)
    state_p = state._buf.data_ptr()  # [scale, hist[0..H-1]]
    d = (nt.GemmDesc * 1)()
    d[0].A, d[0].scale_a, d[0].B, d[0].scale_b, d[0].D = (a.data_ptr(), ma.scale.data_ptr(), b.data_ptr(),
                                                          mb.scale.data_ptr(), out.data_ptr())
    d[0].M, d[0].N, d[0].K = M, N, K
    d[0].fmt_a, d[0].fmt_b, d[0].d_dtype, d[0].accumulate = _FMT[ma.dtype], _FMT[mb.dtype], _OUT_FMT[dtype], 0
    d[0].scale_d, d[0].D_t, d[0].amax_workspace = state_p, nt.ptr(out_t), ws.data_ptr()
    d[0].b_transposed, d[0].a_transposed = int(bt), int(at)
    if bias is not None:
        d[0].bias, d[0].bias_dtype = bias.data_ptr(), nt.TORCH_TO_NT[bias.dtype]
    nt.check(nt.lib.ntfp8_gemm_batch(d, 1, st), "ntfp8_gemm_batch")
    nt.check(nt.lib.ntfp8_amax_finalize(ws.data_ptr(), _FMT[dtype], state.margin, state_p, state_p + 4, state.history_len,
                                        scalars.data_ptr(), scalars.data_ptr() + 4, st), "ntfp8_amax_finalize")
    meta = FP8Meta(scalars[0], scalars[1], dtype)
    obj = torch.Tensor._make_subclass(FP8Tensor, out)
    obj.fp8_meta = meta
    if out_t is not None:
        t = torch.Tensor._make_subclass(FP8Tensor, out_t)
        t.fp8_meta = meta
        obj._transposed = t
    return obj


# Module switch: False makes every GEMM use materialised transposed copies (the reference's way, kernel.py:43-44).
READ_B_TRANSPOSED = True


def b_transposed_supported(M: int, N: int, K: int) -> bool:
    """Whether the library reads the B operand of D[M,N] = A[M,K] . B[N,K]^T from its transpose, a [K, N] tensor
    (`ntfp8_gemm_desc.b_transposed`): the condition stated in include/ntfp8.h."""
    return (READ_B_TRANSPOSED and N % 16 == 0 and K % 16 == 0 and M > 128 and N > 128 and K >= 256
            and (M + 256) * K < 2 ** 31 and (N + 256) * K < 2 ** 31)


# Module switch: False makes wgrad GEMMs take a materialised transpose of the output gradient (kernel.py:44).
READ_A_TRANSPOSED = True


def a_transposed_supported(M: int, N: int, K: int) -> bool:
    """Whether the library reads BOTH operands of D[M,N] = A[M,K] . B[N,K]^T from their transposes, [K, M] and [K, N]
    tensors (`ntfp8_gemm_desc.a_transposed` next to `b_transposed`): the wgrad form, dW = dY^T . X with dY[tokens, out]
    and X[tokens, in] as they are."""
    return READ_A_TRANSPOSED and M % 16 == 0 and b_transposed_supported(M, N, K)


def needs_transposed_copy(rows: int, cols: int, other: int = 4096) -> bool:
    """Whether a [rows, cols] fp8 tensor that a backward GEMM reduces over its rows (the weight in dgrad, the input in
    wgrad; src/nanotron/fp8/linear.py:104-109) should be quantised together with its transposed copy: only if the
    library cannot read it as it is.  `other` is the GEMM's third dimension (tokens for the weight, out_features
    for the input), assumed large when not known yet; a copy that turns out to be needed after all is made on demand."""
    return not b_transposed_supported(other, cols, rows)


def _gemm_nt_batch(problems):
    """Several independent `_gemm_nt` problems, given as tuples (a, b, out_dtype, accumulate_into[, b_transposed[,
    bias[, a_transposed]]]), in one call of the library: GEMMs with the same operand formats share launches.  With
    `b_transposed` the tensor `b` is the [K, N] transpose of the operand, with `a_transposed` the tensor `a` its [K, M]
    transpose.  Returns the outputs in order."""
    descs = (nt.GemmDesc * len(problems))()
    outs, keep = [], []
    dev = problems[0][0].device
    for d, prob in zip(descs, problems):
        a, b, out_dtype, accumulate_into = prob[:4]
        bt = bool(prob[4]) if len(prob) > 4 else False
        bias = prob[5] if len(prob) > 5 else None
        at = bool(prob[6]) if len(prob) > 6 else False
        assert a.dim() == 2 and b.dim() == 2 and a.shape[0 if at else 1] == b.shape[0 if bt else 1], \
            (tuple(a.shape), tuple(b.shape), bt, at)
        assert a.device == dev and b.device == dev
        K, M = a.shape if at else (a.shape[1], a.shape[0])
        N = b.shape[1 if bt else 0]
        a, ma = _bytes_and_meta(a)
        b, mb = _bytes_and_meta(b)
        if accumulate_into is not None:
            assert accumulate_into.dtype == torch.float32 and accumulate_into.shape == (M, N)
            assert accumulate_into.is_contiguous() and accumulate_into.device == dev
            out, acc = accumulate_into, 1
        else:
            out, acc = torch.empty((M, N), dtype=out_dtype, device=dev), 0
        if bias is not None:
            bias = _check_bias(bias, N, dev)
            d.bias, d.bias_dtype = bias.data_ptr(), nt.TORCH_TO_NT[bias.dtype]
        d.A, d.scale_a, d.B, d.scale_b, d.D = a.data_ptr(), ma.scale.data_ptr(), b.data_ptr(), mb.scale.data_ptr(), out.data_ptr()
        d.M, d.N, d.K = M, N, K
        d.fmt_a, d.fmt_b, d.d_dtype, d.accumulate = _FMT[ma.dtype], _FMT[mb.dtype], nt.TORCH_TO_NT[out.dtype], acc
        d.b_transposed = 1 if bt else 0
        d.a_transposed = 1 if at else 0
        outs.append(out)
        keep.append((a, b, bias))
    nt.check(nt.lib.ntfp8_gemm_batch(descs, len(problems), nt.stream_ptr(dev)), "ntfp8_gemm_batch")
    return outs


def _operands(mat_a: FP8Tensor, transpose_a: bool, mat_b: FP8Tensor, transpose_b: bool,
              accumulate_into: Optional[torch.Tensor] = None, allow_bt: bool = True):
    """(A, B, b_transposed, a_transposed) of the library's D = A . B^T for the reference's D = op_b(B) . op_a(A)
    (kernel.py:43-44).

    Where the reference transposes mat_a (tex.fp8_transpose, kernel.py:43) the library can read it as it is
    (`b_transposed`): that is taken when mat_a carries no transposed copy yet and the shape qualifies; otherwise the
    copy is used (and made, once, if it does not exist).  The same for mat_b (kernel.py:44, `a_transposed`), which the
    library serves next to an untransposed mat_a: the wgrad form."""
    assert mat_a.device != torch.device("cpu") and mat_b.device != torch.device("cpu"), \
        "The tensors must be on a CUDA device in order to use the FP8 kernel!!"
    assert hasattr(mat_a, "fp8_meta") and hasattr(mat_b, "fp8_meta"), "operands must be FP8Tensors"
    if transpose_a:
        return (mat_b.transposed() if transpose_b else mat_b), mat_a, False, False
    aligned = all(t is None or t.data_ptr() % 16 == 0 for t in (mat_a, mat_b, accumulate_into))   # 16-byte loads / stores
    plain_a = allow_bt and getattr(mat_a, "_transposed", None) is None and mat_a.dim() == 2 and mat_a.is_contiguous() and aligned
    if transpose_b:
        # D[cols of mat_b, cols of mat_a], reduction over the rows of both
        if plain_a and getattr(mat_b, "_transposed", None) is None and mat_b.dim() == 2 and mat_b.is_contiguous() and \
                a_transposed_supported(mat_b.shape[1], mat_a.shape[1], mat_a.shape[0]):
            return mat_b, mat_a, True, True
        b_ = mat_b.transposed()
    else:
        b_ = mat_b   # the library's A: K-contiguous
    if plain_a and b_.data_ptr() % 16 == 0 and b_transposed_supported(b_.shape[0], mat_a.shape[1], mat_a.shape[0]):
        return b_, mat_a, True, False
    return b_, mat_a.transposed(), False, False


@torch.no_grad()
def fp8_matmul_pair(first: dict, second: dict):
    """Two independent `fp8_matmul_kernel` calls (keyword dictionaries of its arguments) issued together, e.g. the
    dgrad and wgrad of a layer (src/nanotron/fp8/linear.py:104-109 issues them one after the other).  Same
    results as two calls; the library lets the two GEMMs share kernel launches."""
    probs = []
    for kw in (first, second):
        acc = kw.get("accumulate_into")
        A, B, bt, at = _operands(kw["mat_a"], kw["transpose_a"], kw["mat_b"], kw["transpose_b"], acc)
        probs.append((A, B, (kw.get("out_dtype") or torch.float32) if acc is None else torch.float32, acc, bt, None, at))
    return _gemm_nt_batch(probs)


@torch.no_grad()
def fp8_matmul_kernel(
    mat_a: FP8Tensor,
    transpose_a: bool,
    mat_b: FP8Tensor,
    transpose_b: bool,
    use_split_accumulator: bool,
    *,
    out_dtype: Union[torch.dtype, DTypes, None] = None,
    accumulate_into: Optional[torch.Tensor] = None,
    out_state: Optional[DelayedScaling] = None,
    out_with_transpose: bool = False,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """D = op_b(B) . op_a(A) * (1/scale_a)(1/scale_b), op_x(X) = X^T if transpose_x else X
    (reference: src/nanotron/fp8/kernel.py:9-70; the operator meaning follows from its fixed
    te_gemm(transa=True, transb=False) call on row-major tensors).  fp32 output unless `out_dtype`
    says otherwise (kernel.py:24,28).  The result has its true shape [rows of op_b(B), cols of
    op_a(A)], which equals the reference's allocation on the square shapes its tests use.

    `use_split_accumulator` selects cuBLASLt's slower, more accurate accumulation on Hopper; CDNA4
    matrix cores always accumulate in fp32, so it is accepted and ignored.
    `accumulate_into` (fp32, contiguous) receives D added in place before any rounding.
    `out_dtype=DTypes.FP8E4M3 / FP8E5M2` returns D as an FP8Tensor ("return an fp8 tensor as output", the TODO at
    src/nanotron/fp8/linear.py:63-64), quantised with the delayed-scaling state `out_state` in the GEMM's epilogue
    and, with `out_with_transpose`, carrying its transposed copy.
    `bias` (one value per column of D, fp32 / fp16 / bf16) is added to the descaled fp32 result before the single
    rounding to the output type: the bias argument of te_gemm that the reference leaves empty (kernel.py:29-32).
    For an fp32 output this equals `D + bias` bit for bit."""
    assert mat_a.device != torch.device("cpu") and mat_b.device != torch.device("cpu"), \
        "The tensors must be on a CUDA device in order to use the FP8 kernel!!"
    assert hasattr(mat_a, "fp8_meta") and hasattr(mat_b, "fp8_meta"), "operands must be FP8Tensors"
    if isinstance(out_dtype, DTypes):
        assert accumulate_into is None, "an fp8 output cannot accumulate"
        # rows of D: the fp8 epilogue stores whole words of 4 rows' worth of the transposed copy
        rows = mat_b.shape[1] if transpose_b else mat_b.shape[0]
        A, B, bt, at = _operands(mat_a, transpose_a, mat_b, transpose_b, None, allow_bt=bias is None and rows % 4 == 0)
        return _gemm_nt_fp8(A, B, out_dtype, out_state, out_with_transpose, bias, bt, at)
    A, B, bt, at = _operands(mat_a, transpose_a, mat_b, transpose_b, accumulate_into, allow_bt=bias is None)
    if bt:
        return _gemm_nt_batch([(A, B, out_dtype or torch.float32, accumulate_into, True, None, at)])[0]
    return _gemm_nt(A, B, out_dtype or torch.float32, accumulate_into, bias)
