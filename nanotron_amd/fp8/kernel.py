from typing import Optional

import torch

from nanotron_amd import _native as nt
from nanotron_amd.fp8.dtypes import DTypes
from nanotron_amd.fp8.tensor import FP8Tensor

_FMT = {DTypes.FP8E4M3: nt.E4M3, DTypes.FP8E5M2: nt.E5M2}


def _gemm_nt(a: FP8Tensor, b: FP8Tensor, out_dtype: torch.dtype, accumulate_into: Optional[torch.Tensor]):
    """D[M,N] = A[M,K] . B[N,K]^T, descaled (te_gemm's TN form, src/nanotron/fp8/kernel.py:46-68)."""
    assert a.dim() == 2 and b.dim() == 2 and a.shape[1] == b.shape[1], (tuple(a.shape), tuple(b.shape))
    M, K = a.shape
    N = b.shape[0]
    dev = a.device
    if not a.is_contiguous():
        a = a.contiguous()
    if not b.is_contiguous():
        b = b.contiguous()
    ma, mb = a.fp8_meta, b.fp8_meta
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


def _gemm_nt_batch(problems):
    """Several independent `_gemm_nt` problems, given as tuples (a, b, out_dtype, accumulate_into), in one call of
    the library: GEMMs with the same operand formats share launches.  Returns the outputs in order."""
    descs = (nt.GemmDesc * len(problems))()
    outs, keep = [], []
    dev = problems[0][0].device
    for d, (a, b, out_dtype, accumulate_into) in zip(descs, problems):
        assert a.dim() == 2 and b.dim() == 2 and a.shape[1] == b.shape[1], (tuple(a.shape), tuple(b.shape))
        assert a.device == dev and b.device == dev
        M, K = a.shape
        N = b.shape[0]
        if not a.is_contiguous():
            a = a.contiguous()
        if not b.is_contiguous():
            b = b.contiguous()
        ma, mb = a.fp8_meta, b.fp8_meta
        if accumulate_into is not None:
            assert accumulate_into.dtype == torch.float32 and accumulate_into.shape == (M, N)
            assert accumulate_into.is_contiguous() and accumulate_into.device == dev
            out, acc = accumulate_into, 1
        else:
            out, acc = torch.empty((M, N), dtype=out_dtype, device=dev), 0
        d.A, d.scale_a, d.B, d.scale_b, d.D = a.data_ptr(), ma.scale.data_ptr(), b.data_ptr(), mb.scale.data_ptr(), out.data_ptr()
        d.M, d.N, d.K = M, N, K
        d.fmt_a, d.fmt_b, d.d_dtype, d.accumulate = _FMT[ma.dtype], _FMT[mb.dtype], nt.TORCH_TO_NT[out.dtype], acc
        outs.append(out)
        keep.append((a, b))
    nt.check(nt.lib.ntfp8_gemm_batch(descs, len(problems), nt.stream_ptr(dev)), "ntfp8_gemm_batch")
    return outs


def _operands(mat_a: FP8Tensor, transpose_a: bool, mat_b: FP8Tensor, transpose_b: bool):
    """(A, B) of the library's D = A . B^T for the reference's D = op_b(B) . op_a(A) (kernel.py:43-44)."""
    assert mat_a.device != torch.device("cpu") and mat_b.device != torch.device("cpu"), \
        "The tensors must be on a CUDA device in order to use the FP8 kernel!!"
    assert hasattr(mat_a, "fp8_meta") and hasattr(mat_b, "fp8_meta"), "operands must be FP8Tensors"
    a_ = mat_a if transpose_a else mat_a.transposed()
    b_ = mat_b.transposed() if transpose_b else mat_b
    return b_, a_


@torch.no_grad()
def fp8_matmul_pair(first: dict, second: dict):
    """Two independent `fp8_matmul_kernel` calls (keyword dictionaries of its arguments) issued together, e.g. the
    dgrad and wgrad of a layer (src/nanotron/fp8/linear.py:104-109 issues them one after the other).  Same
    results as two calls; the library lets the two GEMMs share kernel launches."""
    probs = []
    for kw in (first, second):
        A, B = _operands(kw["mat_a"], kw["transpose_a"], kw["mat_b"], kw["transpose_b"])
        acc = kw.get("accumulate_into")
        probs.append((A, B, (kw.get("out_dtype") or torch.float32) if acc is None else torch.float32, acc))
    return _gemm_nt_batch(probs)


@torch.no_grad()
def fp8_matmul_kernel(
    mat_a: FP8Tensor,
    transpose_a: bool,
    mat_b: FP8Tensor,
    transpose_b: bool,
    use_split_accumulator: bool,
    *,
    out_dtype: Optional[torch.dtype] = None,
    accumulate_into: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """D = op_b(B) . op_a(A) * (1/scale_a)(1/scale_b), op_x(X) = X^T if transpose_x else X
    (reference: src/nanotron/fp8/kernel.py:9-70; the operator meaning follows from its fixed
    te_gemm(transa=True, transb=False) call on row-major tensors).  fp32 output unless `out_dtype`
    says otherwise (kernel.py:24,28).  The result has its true shape [rows of op_b(B), cols of
    op_a(A)], which equals the reference's allocation on the square shapes its tests use.

    `use_split_accumulator` selects cuBLASLt's slower, more accurate accumulation on Hopper; CDNA4
    matrix cores always accumulate in fp32, so it is accepted and ignored.
    `accumulate_into` (fp32, contiguous) receives D added in place before any rounding."""
    assert mat_a.device != torch.device("cpu") and mat_b.device != torch.device("cpu"), \
        "The tensors must be on a CUDA device in order to use the FP8 kernel!!"
    assert hasattr(mat_a, "fp8_meta") and hasattr(mat_b, "fp8_meta"), "operands must be FP8Tensors"
    a_ = mat_a if transpose_a else mat_a.transposed()  # kernel.py:43
    b_ = mat_b.transposed() if transpose_b else mat_b  # kernel.py:44
    return _gemm_nt(b_, a_, out_dtype or torch.float32, accumulate_into)
