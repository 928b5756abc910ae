"""The four functions of Transformer Engine's pybind module that nanotron's FP8 path calls
(`import transformer_engine_extensions as tex`), served by libntfp8.so with TE's own argument lists:

    tex.cast_to_fp8(input, scale, amax, scale_inv, otype)            src/nanotron/fp8/tensor.py:65
    tex.cast_from_fp8(input, scale_inv, itype, otype)                src/nanotron/fp8/tensor.py:74
    tex.fp8_transpose(input, dtype)                                  src/nanotron/fp8/kernel.py:43-44
    tex.te_gemm(A, A_scale_inverse, A_type, transa, B, B_scale_inverse, B_type, transb, D, D_scale, D_type,
                D_amax, bias, bias_type, pre_gelu_out, grad, workspace, workspace_size, accumulate,
                use_split_accumulator, math_sm_count)                src/nanotron/fp8/kernel.py:46-68
    tex.DType                                                        src/nanotron/fp8/tensor.py:55, kernel.py:28

`install()` registers this module as `transformer_engine_extensions` (and an empty `transformer_engine`), so that
the reference's `src/nanotron/fp8/*.py` run unedited on an MI355X: their call sites keep passing
`meta.inverse_scale`, the dummy `scale_inv = 1.0` and the empty bias / amax / scale tensors, and every one of those
arguments is honoured here as Transformer Engine honours it.

Everything is asynchronous on torch's current stream; errors of the native library surface as RuntimeError, as
TE's C++ exceptions do.
"""
from __future__ import annotations

import sys
import types

import torch

from nanotron_amd import _native as nt
from nanotron_amd.fp8.dtypes import DType

_FP8 = {DType.kFloat8E4M3: nt.E4M3, DType.kFloat8E5M2: nt.E5M2}
_FP8_OUT = {DType.kFloat8E4M3: nt.OUT_E4M3, DType.kFloat8E5M2: nt.OUT_E5M2}
_HP = {DType.kFloat32: torch.float32, DType.kFloat16: torch.float16, DType.kBFloat16: torch.bfloat16}


def _fmt(t) -> int:
    try:
        return _FP8[DType(int(t))]
    except (KeyError, ValueError):
        raise RuntimeError(f"{t!r} is not an FP8 type (kFloat8E4M3 / kFloat8E5M2)") from None


def _scalar(t: torch.Tensor, dev, what: str) -> torch.Tensor:
    """A one-element fp32 tensor on `dev` (TE takes device tensors; a host scalar is moved over)."""
    if not isinstance(t, torch.Tensor) or t.numel() != 1:
        raise RuntimeError(f"{what} must be a tensor with one element")
    if t.device != dev or t.dtype != torch.float32:
        t = t.to(device=dev, dtype=torch.float32)
    return t


def cast_to_fp8(input: torch.Tensor, scale: torch.Tensor, amax: torch.Tensor, scale_inv: torch.Tensor, otype) -> torch.Tensor:
    """out = saturating_rne_fp8(input * scale) as uint8, same shape; `amax` (one element, updated in place) becomes
    max(amax, max|input|); `scale_inv` (one element, in place) becomes 1 / scale."""
    if input.device.type != "cuda":
        raise RuntimeError("cast_to_fp8: input must be a device tensor")
    if input.dtype not in nt.TORCH_TO_NT:
        raise RuntimeError(f"cast_to_fp8: unsupported input type {input.dtype}")
    x = input.detach().contiguous()
    dev = x.device
    out = torch.empty(x.shape, dtype=torch.uint8, device=dev)
    if x.numel() == 0:
        return out
    sc = _scalar(scale, dev, "scale")

    def in_place(t, what):
        # updated in place when it is a one-element fp32 device tensor; anything else (the reference hands over
        # fresh dummies, tensor.py:64) cannot be seen by the caller afterwards and is left alone
        if isinstance(t, torch.Tensor) and t.numel() == 1 and t.device == dev and t.dtype == torch.float32 and t.is_contiguous():
            return t
        return None

    am, si = in_place(amax, "amax"), in_place(scale_inv, "scale_inv")
    ws, st = nt.workspace_and_stream(dev)
    nt.check(nt.lib.ntfp8_te_cast_to_fp8(x.data_ptr(), nt.TORCH_TO_NT[x.dtype], x.numel(), sc.data_ptr(), nt.ptr(am),
                                         nt.ptr(si), _fmt(otype), out.data_ptr(), ws.data_ptr(), st), "cast_to_fp8")
    return out


def cast_from_fp8(input: torch.Tensor, scale_inv: torch.Tensor, itype, otype) -> torch.Tensor:
    """out = otype(fp32(fp8 bytes) * scale_inv)."""
    if input.device.type != "cuda":
        raise RuntimeError("cast_from_fp8: input must be a device tensor")
    try:
        out_dtype = _HP[DType(int(otype))]
    except (KeyError, ValueError):
        raise RuntimeError(f"cast_from_fp8: unsupported output type {otype!r}") from None
    q = input.detach().as_subclass(torch.Tensor).contiguous()
    dev = q.device
    out = torch.empty(q.shape, dtype=out_dtype, device=dev)
    if q.numel():
        si = _scalar(scale_inv, dev, "scale_inv")
        nt.check(nt.lib.ntfp8_cast_from_fp8_scale_inv(q.data_ptr(), _fmt(itype), si.data_ptr(), q.numel(), out.data_ptr(),
                                                      nt.TORCH_TO_NT[out_dtype], nt.stream_ptr(dev)), "cast_from_fp8")
    return out


def fp8_transpose(input: torch.Tensor, dtype) -> torch.Tensor:
    """[rows, cols] bytes -> contiguous [cols, rows] bytes."""
    _fmt(dtype)
    if input.dim() != 2:
        raise RuntimeError("fp8_transpose: input must be 2-D")
    q = input.detach().as_subclass(torch.Tensor).contiguous()
    rows, cols = q.shape
    out = torch.empty((cols, rows), dtype=torch.uint8, device=q.device)
    if q.numel():
        nt.check(nt.lib.ntfp8_transpose(q.data_ptr(), rows, cols, out.data_ptr(), nt.stream_ptr(q.device)), "fp8_transpose")
    return out


def te_gemm(A: torch.Tensor, A_scale_inverse: torch.Tensor, A_type, transa: bool,
            B: torch.Tensor, B_scale_inverse: torch.Tensor, B_type, transb: bool,
            D: torch.Tensor, D_scale: torch.Tensor, D_type, D_amax: torch.Tensor,
            bias: torch.Tensor, bias_type, pre_gelu_out: torch.Tensor, grad: bool,
            workspace: torch.Tensor, workspaceSize: int, accumulate: bool, use_split_accumulator: bool,
            math_sm_count: int = 0) -> None:
    """cuBLASLt's column-major GEMM on row-major torch tensors, written into D:
        transa=True,  transb=False:  D[B.rows, A.rows] = B . A^T        (the form the reference issues)
        transa=False, transb=False:  D[B.rows, A.cols] = B . A
        transa=False, transb=True:   D[B.cols, A.cols] = B^T . A        (the wgrad form)
        transa=True,  transb=True:   D[B.cols, A.rows] = B^T . A^T
    times A_scale_inverse * B_scale_inverse, fp32 accumulation, plus `bias` (one value per column of D) if it is
    not empty, one rounding to D's type; `accumulate` adds into an fp32 D.  With an fp8 `D_type`, D receives
    sat_rne_fp8(result * D_scale) and D_amax max(D_amax, max|result|).

    Every form is served for every shape.  The library reads an operand that is not contiguous along the reduction
    index as it lies in memory where its big kernel can (no bias, N a multiple of 16, M and N above 128, K >= 256,
    operands below 2 GiB; a transposed B only next to a transposed A); elsewhere the operand is transposed first
    (ntfp8_transpose) and the K-contiguous form is issued, which has no such limits.  Not served: `grad` together with
    a bias (the bias-gradient epilogue) and a non-empty `pre_gelu_out`.  `workspace`, `use_split_accumulator` and
    `math_sm_count` have no meaning here: the kernels need no workspace and the matrix cores always accumulate in fp32."""
    if grad and bias is not None and bias.numel() > 0:
        raise RuntimeError("te_gemm: the bias-gradient epilogue (grad=True with a bias) is not supported")
    if pre_gelu_out is not None and pre_gelu_out.numel() > 0:
        raise RuntimeError("te_gemm: the GELU epilogue is not supported")
    if A.dim() != 2 or B.dim() != 2:
        raise RuntimeError("te_gemm: operands must be 2-D")
    a = A.detach().as_subclass(torch.Tensor).contiguous()
    b = B.detach().as_subclass(torch.Tensor).contiguous()
    dev = a.device
    M, K = (b.shape[1], b.shape[0]) if transb else b.shape   # rows of D, reduction length
    if transa:
        N, Ka = a.shape
    else:
        Ka, N = a.shape
    if Ka != K:
        raise RuntimeError(f"te_gemm: reduction lengths differ ({tuple(A.shape)}, transa={transa}; {tuple(B.shape)})")
    if tuple(D.shape) != (M, N) or not D.is_contiguous() or D.device != dev:
        raise RuntimeError(f"te_gemm: D must be a contiguous [{M}, {N}] tensor on {dev}")
    sa = _scalar(A_scale_inverse, dev, "A_scale_inverse")
    sb = _scalar(B_scale_inverse, dev, "B_scale_inverse")
    d = (nt.GemmDesc * 1)()
    p = d[0]
    # the library computes D = A_lib . B_lib^T with A_lib = B (rows of D), B_lib = A
    p.A, p.scale_a, p.fmt_a = b.data_ptr(), sb.data_ptr(), _fmt(B_type)
    p.B, p.scale_b, p.fmt_b = a.data_ptr(), sa.data_ptr(), _fmt(A_type)
    p.b_transposed = 0 if transa else 1
    p.a_transposed = 1 if transb else 0
    has_bias = bias is not None and bias.numel() > 0
    # forms the library does not read in place: transposed copies and the K-contiguous form
    copies = (p.a_transposed and not p.b_transposed) or (has_bias and (p.a_transposed or p.b_transposed))

    def use_copies():
        nonlocal a, b
        if p.b_transposed:
            a = fp8_transpose(a, A_type)
        if p.a_transposed:
            b = fp8_transpose(b, B_type)
        p.A, p.B, p.a_transposed, p.b_transposed = b.data_ptr(), a.data_ptr(), 0, 0
        keep.extend([a, b])
    p.scales_are_inverse = 1
    p.D, p.M, p.N, p.K = D.data_ptr(), M, N, K
    p.accumulate = 1 if accumulate else 0
    keep = [a, b, sa, sb]
    if copies:
        use_copies()
    st = nt.stream_ptr(dev)
    fp8_out = D.dtype == torch.uint8
    if fp8_out:
        try:
            p.d_dtype = _FP8_OUT[DType(int(D_type))]
        except (KeyError, ValueError):
            raise RuntimeError("te_gemm: a uint8 D needs an FP8 D_type") from None
        ds = _scalar(D_scale, dev, "D_scale")
        p.scale_d = ds.data_ptr()
        keep.append(ds)
        want_amax = isinstance(D_amax, torch.Tensor) and D_amax.numel() == 1
        if want_amax:
            ws, _ = nt.workspace_and_stream(dev)
            p.amax_workspace = ws.data_ptr()
    else:
        if D.dtype not in nt.TORCH_TO_NT:
            raise RuntimeError(f"te_gemm: unsupported output type {D.dtype}")
        p.d_dtype = nt.TORCH_TO_NT[D.dtype]
    if has_bias:
        if bias.numel() != N or bias.dtype not in nt.TORCH_TO_NT:
            raise RuntimeError(f"te_gemm: bias must hold {N} fp32 / fp16 / bf16 values")
        bb = bias.detach().to(dev).contiguous()
        p.bias, p.bias_dtype = bb.data_ptr(), nt.TORCH_TO_NT[bb.dtype]
        keep.append(bb)
    rc = nt.lib.ntfp8_gemm_batch(d, 1, st)
    if rc == nt.ERR_UNSUPPORTED and (p.a_transposed or p.b_transposed):
        use_copies()   # a shape the in-place reads do not serve (refused before anything was launched)
        rc = nt.lib.ntfp8_gemm_batch(d, 1, st)
    nt.check(rc, "te_gemm")
    if fp8_out and want_amax:
        # the maxima the epilogue left in the workspace -> max(D_amax, max|result|); no history, scale untouched
        am = D_amax if (D_amax.device == dev and D_amax.dtype == torch.float32) else None
        tmp = am if am is not None else torch.zeros(1, dtype=torch.float32, device=dev)
        prev = tmp.clone()
        nt.check(nt.lib.ntfp8_amax_finalize(ws.data_ptr(), nt.E4M3 if p.d_dtype == nt.OUT_E4M3 else nt.E5M2, 0, ds.data_ptr(),
                                            None, 0, tmp.data_ptr(), None, st), "te_gemm (amax)")
        torch.maximum(tmp, prev, out=tmp)


def install() -> types.ModuleType:
    """Register this module under the names the reference imports (`transformer_engine_extensions`, and a bare
    `transformer_engine` package for the `import transformer_engine as te  # noqa` lines).  Returns the module."""
    me = sys.modules[__name__]
    sys.modules.setdefault("transformer_engine", types.ModuleType("transformer_engine"))
    sys.modules["transformer_engine_extensions"] = me
    return me
