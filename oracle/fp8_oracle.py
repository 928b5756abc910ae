"""CPU oracle for the nanotron.fp8 hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, with torch-CPU / numpy arithmetic, what the reference's
FP8 linear path computes.  It is imported only by tests/, by
__graft_entry__.smoke() and by bench.py's cpu_baseline leg, and only as the
checker: the product (nanotron_amd) never imports it and has no CPU fallback.

Every function cites the reference lines it follows (paths relative to the
reference checkout, src/nanotron/fp8/...).  The arithmetic of the reference's
cast / dequant / transpose / GEMM lives in NVIDIA Transformer Engine
(`transformer_engine_extensions`, imported at fp8/tensor.py:2-3, un-vendored and
un-pinned in the reference's pyproject.toml), so for those functions the oracle
restates the published semantics of TE's `cast_to_fp8`, `cast_from_fp8`,
`fp8_transpose` and `te_gemm` (OCP FP8 formats, saturating round-to-nearest-even,
fp32 accumulation, one descale multiply) anchored on the reference's call sites.

Pinning status (what independent evidence each function is checked against in
tests/test_oracle.py):

  amax                      definition max|x|; exact, order free.           PINNED
  update_scaling_factor     closed form 2**floor(log2(fp8_max/amax)); known
                            answers 256.0 / 32768.0 that fp8/linear.py:33-42
                            evaluates; exhaustive bf16 + fp16 amax sweep vs
                            frexp; invariants.                              PINNED
  cast_to_fp8               OCP FP8 spec decode table + independent nearest-
                            value/ties-to-even search (numpy) + independent
                            integer-only C encoder (oracle/fp8_oracle.c);
                            exhaustive over all bf16 bit patterns.          PINNED
                            Sign of a NaN *generated* by 0*inf: parity unpinned.
  cast_from_fp8             decode table x power of two.                    PINNED
  fp8_transpose             byte permutation.                               PINNED
  gemm                      fp64 matmul cross-check; integer-valued operands
                            where every partial sum is exact in fp32.       PINNED
                            (fp32 accumulation ORDER inside TE/cuBLASLt is
                            unknowable: parity is the stated rel-L2 <= 1e-3.)
  DelayedScaling            bookkeeping defined by this build (the reference
                            has no amax history); known-answer sequences.   PINNED
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional, Tuple

import numpy as np
import torch

E4M3 = "e4m3"
E5M2 = "e5m2"

# fp8/constants.py:18  DTYPE_TO_FP8_MAX
FP8_MAX = {E4M3: 448.0, E5M2: 57344.0}
TORCH_FP8 = {E4M3: torch.float8_e4m3fn, E5M2: torch.float8_e5m2}
# fp8/constants.py:8
INITIAL_SCALING_FACTOR = 1.0


# --------------------------------------------------------------------------- amax
def amax(x: torch.Tensor) -> torch.Tensor:
    """fp8/tensor.py:25  `amax = tensor.abs().max().clone()`, returned as 0-dim fp32.

    bf16/fp16 -> fp32 is exact, so taking the max before or after the upcast is the
    same number.  NaN propagates (torch.max semantics); an empty tensor raises.
    """
    return x.detach().abs().max().to(torch.float32).clone()


# --------------------------------------------------------------------------- scale
def update_scaling_factor(
    amax_: torch.Tensor, scaling_factor: torch.Tensor, fmt: str, margin: float = 0
) -> torch.Tensor:
    """fp8/tensor.py:77-105, the seven tensor ops of `_inner` restated one to one
    (TorchScript only fuses them; the arithmetic is the eager one)."""
    assert amax_.dtype == torch.float32  # fp8/tensor.py:84
    assert scaling_factor.dtype == torch.float32  # fp8/tensor.py:86
    fp8_max = torch.tensor(FP8_MAX[fmt], dtype=torch.float32)  # fp8/tensor.py:90
    ratio = fp8_max / amax_  # :97
    exp = torch.floor(torch.log2(ratio)) - margin  # :98
    new_sf = torch.round(torch.pow(2, torch.abs(exp)))  # :99
    new_sf = torch.where(amax_ > 0.0, new_sf, scaling_factor)  # :100
    new_sf = torch.where(torch.isfinite(amax_), new_sf, scaling_factor)  # :101
    new_sf = torch.where(exp < 0, 1 / new_sf, new_sf)  # :102
    return new_sf.to(torch.float32)


def scale_closed_form(amax_value: float, old_scale: float, fmt: str, margin: int = 0) -> float:
    """Independent statement of the same function by exponent extraction, used to pin
    update_scaling_factor.  Works in exact arithmetic on the fp32 quotient:
    scale = 2**(floor(log2(q)) - margin), q = fl32(fp8_max / amax).

    The literal formula goes through a *rounded* fp32 log2, so when q sits within a
    few ulps below a power of two 2**k (|k| >= 2) log2f(q) rounds up to k and the
    literal result is 2**k, not 2**(k-1).  The code below reproduces that by rounding
    the double-precision log2 to fp32 before taking the floor."""
    a = np.float32(amax_value)
    if np.isinf(a):
        # literal quirk of tensor.py:97-102: ratio = 0, log2 = -inf, so the "keep the old
        # scale" branch (:101) is followed by the reciprocal branch (:102, exp < 0).  The
        # reference only ever passes old = 1.0, where 1/old == old.
        return float(np.float32(1.0) / np.float32(old_scale))
    if not (a > 0):
        return float(np.float32(old_scale))
    with np.errstate(over="ignore", divide="ignore"):
        q = np.float32(FP8_MAX[fmt]) / a
    if np.isinf(q):
        return float("inf")
    l = np.float32(math.log2(float(q)))  # correctly rounded fp32 log2 (double log2, one rounding)
    e = int(math.floor(float(l))) - int(margin)
    if abs(e) >= 128:
        return 0.0 if e < 0 else float("inf")
    return float(np.float32(2.0) ** np.float32(e))


# --------------------------------------------------------------------------- cast
def cast_to_fp8(x: torch.Tensor, scale: torch.Tensor, fmt: str) -> torch.Tensor:
    """fp8/tensor.py:60-65 -> tex.cast_to_fp8(tensor, scale, amax, scale_inv, otype):
    out[i] = saturating_rne_fp8( fp32(x[i]) * scale ).  One fp32 multiply, clamp to
    +-fp8_max with NaN passing through, round-to-nearest-even to the OCP format.
    Returns uint8 bytes of the same shape (tests/fp8/test_tensor.py:23)."""
    y = x.detach().to(torch.float32) * scale.to(torch.float32)
    m = FP8_MAX[fmt]
    y = torch.clamp(y, -m, m)
    return y.to(TORCH_FP8[fmt]).view(torch.uint8)


def decode_table(fmt: str) -> np.ndarray:
    """All 256 byte values decoded from the OCP FP8 spec (no torch involved):
    e4m3fn: bias 7, no Inf, NaN = S.1111.111; e5m2: bias 15, IEEE-like Inf/NaN."""
    out = np.zeros(256, dtype=np.float64)
    ebits, mbits, bias = (4, 3, 7) if fmt == E4M3 else (5, 2, 15)
    for b in range(256):
        s = -1.0 if b & 0x80 else 1.0
        e = (b >> mbits) & ((1 << ebits) - 1)
        m = b & ((1 << mbits) - 1)
        if fmt == E4M3 and e == 15 and m == 7:
            v = float("nan")
        elif fmt == E5M2 and e == 31:
            v = float("inf") if m == 0 else float("nan")
        elif e == 0:
            v = m / (1 << mbits) * 2.0 ** (1 - bias)
        else:
            v = (1 + m / (1 << mbits)) * 2.0 ** (e - bias)
        out[b] = s * v
    return out


def cast_to_fp8_search(y: np.ndarray, fmt: str) -> np.ndarray:
    """Independent encoder: for each already-scaled fp32 value pick the nearest finite
    representable magnitude, ties to the code with an even mantissa, saturating at
    fp8_max; NaN -> sign|0x7F.  Pure search over the spec decode table."""
    tab = decode_table(fmt)
    max_code = 0x7E if fmt == E4M3 else 0x7B
    mags = tab[: max_code + 1]  # monotone increasing finite magnitudes, codes 0..max_code
    y64 = y.astype(np.float64).ravel()
    sign = np.signbit(y64).astype(np.uint8) << 7
    a = np.abs(y64)
    nan = np.isnan(a)
    a = np.where(nan, 0.0, np.minimum(a, mags[-1]))
    hi = np.searchsorted(mags, a, side="left")  # first code with mag >= a
    hi = np.minimum(hi, max_code)
    lo = np.maximum(hi - 1, 0)
    dlo = a - mags[lo]
    dhi = mags[hi] - a
    pick_hi = (dhi < dlo) | ((dhi == dlo) & ((hi & 1) == 0))
    code = np.where(pick_hi, hi, lo).astype(np.uint8)
    code = np.where(nan, np.uint8(0x7F), code)
    return (code | sign).reshape(y.shape)


def cast_from_fp8(q: torch.Tensor, scale: torch.Tensor, fmt: str, out_dtype: torch.dtype) -> torch.Tensor:
    """fp8/tensor.py:68-74 -> tex.cast_from_fp8(tensor, meta.inverse_scale, itype, otype):
    out = otype( fp32(fp8) * (1/scale) );  1/scale as fp8/meta.py:36-37."""
    inv = 1 / scale.to(torch.float32)
    return (q.view(TORCH_FP8[fmt]).to(torch.float32) * inv).to(out_dtype)


def fp8_transpose(q: torch.Tensor) -> torch.Tensor:
    """fp8/kernel.py:43-44 -> tex.fp8_transpose: [M,N] bytes -> contiguous [N,M]."""
    assert q.dim() == 2
    return q.t().contiguous()


def upcast(q: torch.Tensor, fmt: str, dtype=torch.float32) -> torch.Tensor:
    return q.view(TORCH_FP8[fmt]).to(dtype)


# --------------------------------------------------------------------------- GEMM
def gemm_nt(
    a: torch.Tensor, fmt_a: str, scale_a: torch.Tensor,
    b: torch.Tensor, fmt_b: str, scale_b: torch.Tensor,
    out_dtype: torch.dtype = torch.float32,
    accumulate_into: Optional[torch.Tensor] = None,
    acc_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """D[M,N] = A[M,K] . B[N,K]^T * (1/scale_a)(1/scale_b): the one GEMM form the
    reference ever issues (fp8/kernel.py:46-68, te_gemm with transa=True,
    transb=False, i.e. both operands contiguous along the reduction dimension),
    fp32 accumulation, fp32 output by default (fp8/kernel.py:24,28).  Operands are
    the fp8 bytes upcast exactly; the scale product is applied once to the sum.
    `accumulate_into` (fp32) restates `fp32_grad.add_(grad)` of
    optim/gradient_accumulator.py:222 done before any rounding."""
    af = upcast(a, fmt_a, acc_dtype)
    bf = upcast(b, fmt_b, acc_dtype)
    alpha = (1 / scale_a.to(torch.float32)) * (1 / scale_b.to(torch.float32))
    d = (af @ bf.t()) * alpha.to(acc_dtype)
    if accumulate_into is not None:
        d = d + accumulate_into.to(acc_dtype)
    return d.to(out_dtype)


def fp8_matmul_kernel(a, fmt_a, scale_a, transpose_a, b, fmt_b, scale_b, transpose_b,
                      out_dtype=torch.float32, acc_dtype=torch.float32):
    """fp8/kernel.py:9-70: D = op_b(B) . op_a(A), where op_x(X) = X^T if transpose_x
    else X, descaled, fp32.  (cuBLASLt 'TN' on column-major views: with row-major
    storage te_gemm(A', transa=True, B', transb=False) yields B'.A'^T; A' = A if
    transpose_a else A^T (kernel.py:43); B' = B^T if transpose_b else B (kernel.py:44).)"""
    a_ = a if transpose_a else fp8_transpose(a)  # kernel.py:43
    b_ = fp8_transpose(b) if transpose_b else b  # kernel.py:44
    # te_gemm: out = B' . A'^T  -> gemm_nt(A=B', B=A')
    return gemm_nt(b_, fmt_b, scale_b, a_, fmt_a, scale_a, out_dtype, None, acc_dtype)


# --------------------------------------------------------------------------- FP8Tensor
@dataclass
class Quantised:
    q: torch.Tensor  # uint8 bytes
    amax: torch.Tensor  # 0-dim fp32: amax of the source tensor
    scale: torch.Tensor  # 0-dim fp32: the scale the bytes were produced with
    fmt: str


def quantise_current(x: torch.Tensor, fmt: str, margin: float = 0) -> Quantised:
    """fp8/tensor.py:25-28: amax of this tensor, scale from it starting at 1.0, cast."""
    a = amax(x)
    s = update_scaling_factor(a, torch.tensor(INITIAL_SCALING_FACTOR, dtype=torch.float32), fmt, margin)
    return Quantised(cast_to_fp8(x, s, fmt), a, s, fmt)


@dataclass
class DelayedScaling:
    """Per tensor-role delayed scaling with an amax history.  NOT in the reference
    (it has no history, fp8/tensor.py:25-28 is current scaling); defined by this
    build's benchmark configs: history length 16, margin 0.

      1. a_t = amax(x_t)
      2. scale used: first use (no finite positive amax recorded yet) -> current
         scaling from a_t exactly as fp8/tensor.py:26; else the stored scale
      3. q_t = cast(x_t, s_t)
      4. hist[1:] = hist[:-1]; hist[0] = a_t
      5. scale <- update_scaling_factor(max(hist), s_t)   (NaN/Inf/0 keep s_t)
    """

    fmt: str
    history_len: int = 16
    margin: float = 0
    hist: torch.Tensor = field(default=None)
    scale: torch.Tensor = field(default=None)
    initialised: bool = False

    def __post_init__(self):
        if self.hist is None:
            self.hist = torch.zeros(self.history_len, dtype=torch.float32)
        if self.scale is None:
            self.scale = torch.tensor(INITIAL_SCALING_FACTOR, dtype=torch.float32)

    def quantise(self, x: torch.Tensor) -> Quantised:
        a = amax(x)
        if not self.initialised:
            s = update_scaling_factor(a, torch.tensor(INITIAL_SCALING_FACTOR, dtype=torch.float32),
                                      self.fmt, self.margin)
        else:
            s = self.scale.clone()
        q = cast_to_fp8(x, s, self.fmt)
        self.hist = torch.cat([a.reshape(1), self.hist[:-1]])
        hmax = self.hist.max()  # NaN-propagating like amax
        self.scale = update_scaling_factor(hmax, s, self.fmt, self.margin)
        if bool(torch.isfinite(a)) and float(a) > 0:
            self.initialised = True
        return Quantised(q, a, s, self.fmt)


# --------------------------------------------------------------------------- FP8Linear
def linear_forward(xq: Quantised, wq: Quantised, out_dtype=torch.float32, acc_dtype=torch.float32):
    """fp8/linear.py:82-84: fp8_matmul_kernel(mat_a=W, transpose_a=True, mat_b=X,
    transpose_b=False)  =>  Y[M,N] = X[M,K] . W[N,K]^T."""
    return fp8_matmul_kernel(wq.q, wq.fmt, wq.scale, True, xq.q, xq.fmt, xq.scale, False, out_dtype, acc_dtype)


def linear_dgrad(gq: Quantised, wq: Quantised, out_dtype=torch.float32, acc_dtype=torch.float32):
    """Intended maths of fp8/linear.py:104-106 (the docstring at linear.py:92-96):
    dX[M,K] = dY[M,N] . W[N,K], via fp8_matmul_kernel(a=W, ta=False, b=dY, tb=False)."""
    return fp8_matmul_kernel(wq.q, wq.fmt, wq.scale, False, gq.q, gq.fmt, gq.scale, False, out_dtype, acc_dtype)


def linear_wgrad(gq: Quantised, xq: Quantised, out_dtype=torch.float32, acc_dtype=torch.float32,
                 accumulate_into=None):
    """Intended maths of fp8/linear.py:107-109: dW[N,K] = dY[M,N]^T . X[M,K], via
    fp8_matmul_kernel(a=X, ta=False, b=dY, tb=True); optional fp32 accumulate
    (optim/gradient_accumulator.py:222)."""
    d = fp8_matmul_kernel(xq.q, xq.fmt, xq.scale, False, gq.q, gq.fmt, gq.scale, True, torch.float32, acc_dtype)
    if accumulate_into is not None:
        d = d + accumulate_into.to(d.dtype)
    return d.to(out_dtype)


def rel_l2(d: torch.Tensor, ref: torch.Tensor) -> float:
    d = d.double()
    ref = ref.double()
    return float((d - ref).norm() / ref.norm().clamp_min(1e-300))


# --------------------------------------------------------------------------- synthetic inputs
def student_t_outlier_tensor(seed: int, shape=(4096, 4096), dtype=torch.bfloat16) -> torch.Tensor:
    """Benchmark config 2 input: 0.5 * Student-t(df=3), 0.01 % of entries replaced by
    +-U(50,500) outliers; numpy PCG64 so the bits are reproducible everywhere."""
    rng = np.random.Generator(np.random.PCG64(seed))
    n = int(np.prod(shape))
    v = (0.5 * rng.standard_t(3, size=n)).astype(np.float32)
    k = max(1, int(round(n * 1e-4)))
    idx = rng.choice(n, size=k, replace=False)
    v[idx] = (rng.uniform(50.0, 500.0, size=k) * rng.choice([-1.0, 1.0], size=k)).astype(np.float32)
    return torch.from_numpy(v).reshape(shape).to(dtype)


def normal_tensor(seed: int, shape, std: float, dtype=torch.bfloat16) -> torch.Tensor:
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(dtype)
