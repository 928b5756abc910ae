"""ctypes binding of libntfp8.so, the C-ABI library declared in include/ntfp8.h.

There is no fallback: if the library is missing the import fails, and every wrapper turns a
non-zero return code into a RuntimeError.
"""
from __future__ import annotations

import ctypes
import os
from typing import Dict, Optional, Tuple

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libntfp8.so")

E4M3, E5M2 = 0, 1
F32, F16, BF16 = 0, 1, 2
OUT_E4M3, OUT_E5M2 = 3, 4  # d_dtype of an fp8 GEMM output
WORKSPACE_BYTES = 2048
STATIC_MAX_TENSORS = 16  # tensors per ntfp8_quantize_delayed_batch_static call
ERR_UNSUPPORTED, ERR_LAUNCH = -5, -6

TORCH_TO_NT = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}

if not os.path.exists(LIB_PATH):
    raise ImportError(
        f"{LIB_PATH} is missing: build the HIP library first (python -m nanotron_amd.build). "
        "nanotron_amd has no CPU or PyTorch fallback for its kernels."
    )

_lib = ctypes.CDLL(LIB_PATH)

_c = ctypes
_vp, _i, _i64, _f = _c.c_void_p, _c.c_int, _c.c_int64, _c.c_float

class GemmDesc(ctypes.Structure):
    """`ntfp8_gemm_desc` of include/ntfp8.h."""
    _fields_ = [("A", _vp), ("scale_a", _vp), ("B", _vp), ("scale_b", _vp), ("D", _vp),
                ("M", _i64), ("N", _i64), ("K", _i64),
                ("fmt_a", _i), ("fmt_b", _i), ("d_dtype", _i), ("accumulate", _i),
                ("scale_d", _vp), ("D_t", _vp), ("amax_workspace", _vp), ("b_transposed", _i),
                ("bias", _vp), ("bias_dtype", _i), ("scales_are_inverse", _i), ("a_transposed", _i)]


class QuantDesc(ctypes.Structure):
    """`ntfp8_quant_desc` of include/ntfp8.h."""
    _fields_ = [("x", _vp), ("x_dtype", _i), ("fmt", _i), ("margin", _i), ("history_len", _i),
                ("rows", _i64), ("cols", _i64),
                ("scale_state", _vp), ("amax_history", _vp), ("amax_out", _vp), ("scale_used_out", _vp),
                ("out", _vp), ("out_t", _vp), ("workspace", _vp)]


SIGNATURES = {
    "ntfp8_version": (_i, []),
    "ntfp8_strerror": (_c.c_char_p, [_i]),
    "ntfp8_amax_scale": (_i, [_vp, _i, _i64, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "ntfp8_update_scaling_factor": (_i, [_vp, _vp, _i, _i, _vp, _i64, _vp]),
    "ntfp8_update_scaling_factor_host": (_f, [_f, _f, _i, _i]),
    "ntfp8_cast_to_fp8": (_i, [_vp, _i, _i64, _i64, _vp, _i, _vp, _vp, _vp]),
    "ntfp8_quantize_current": (_i, [_vp, _i, _i64, _i64, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp]),
    "ntfp8_quantize_first_use": (_i, [_vp, _i, _i64, _i64, _i, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "ntfp8_quantize_delayed": (_i, [_vp, _i, _i64, _i64, _i, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp]),
    "ntfp8_quantize_delayed_batch": (_i, [_c.POINTER(QuantDesc), _i, _vp]),
    "ntfp8_quantize_delayed_batch_static": (_i, [_c.POINTER(QuantDesc), _i, _vp]),
    "ntfp8_static_init": (_i, [_vp]),
    "ntfp8_quantize_delayed_dual": (_i, [_vp, _i, _i64, _i, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "ntfp8_te_cast_to_fp8": (_i, [_vp, _i, _i64, _vp, _vp, _vp, _i, _vp, _vp, _vp]),
    "ntfp8_cast_from_fp8": (_i, [_vp, _i, _vp, _i64, _vp, _i, _vp]),
    "ntfp8_cast_from_fp8_scale_inv": (_i, [_vp, _i, _vp, _i64, _vp, _i, _vp]),
    "ntfp8_transpose": (_i, [_vp, _i64, _i64, _vp, _vp]),
    "ntfp8_gemm": (_i, [_vp, _i, _vp, _vp, _i, _vp, _vp, _i, _i64, _i64, _i64, _i, _vp]),
    "ntfp8_gemm_batch": (_i, [_c.POINTER(GemmDesc), _i, _vp]),
    "ntfp8_amax_finalize": (_i, [_vp, _i, _i, _vp, _vp, _i, _vp, _vp, _vp]),
    "ntfp8_stream_probe": (_i, [_i, _vp, _i64, _vp, _vp]),
}

for _name, (_res, _args) in SIGNATURES.items():
    _fn = getattr(_lib, _name)  # AttributeError here = library / header mismatch
    _fn.restype = _res
    _fn.argtypes = _args

lib = _lib


def strerror(code: int) -> str:
    return _lib.ntfp8_strerror(code).decode()


def check(code: int, what: str) -> None:
    if code != 0:
        if code == ERR_LAUNCH:
            # whatever went wrong at the launch, nothing may be assumed about the reduction workspaces any more (they
            # must be all zero between launches): drop them, the next call gets fresh zeroed ones
            _workspaces.clear()
            _pools.clear()
        raise RuntimeError(f"{what} failed: {strerror(code)} (code {code})")


def version() -> int:
    return _lib.ntfp8_version()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device: torch.device) -> int:
    """hipStream_t of torch's current stream on `device` (the raw accessor costs a fraction of a microsecond,
    the Stream object several)."""
    if _raw_stream is not None:
        return _raw_stream(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


_workspaces: Dict[Tuple[int, int], torch.Tensor] = {}


def workspace_and_stream(device: torch.device) -> Tuple[torch.Tensor, int]:
    """(zero-initialised reduction workspace, stream pointer) for torch's current stream on `device`; one
    workspace per (device, stream): kernels leave it zero."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    st = stream_ptr(device)
    ws = _workspaces.get((idx, st))
    if ws is None:
        ws = torch.zeros(WORKSPACE_BYTES // 4, dtype=torch.int32, device=device)
        _workspaces[(idx, st)] = ws
    return ws, st


_pools: Dict[Tuple[int, int], torch.Tensor] = {}


def workspace_pool(device: torch.device, count: int) -> Tuple[torch.Tensor, int]:
    """([>= count, WORKSPACE_BYTES / 4] zero-initialised workspaces, stream pointer) for torch's current stream on
    `device`: one workspace per tensor of a batched call (kernels leave them zero)."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    st = stream_ptr(device)
    pool = _pools.get((idx, st))
    if pool is None or pool.shape[0] < count:
        pool = torch.zeros(max(count, 16), WORKSPACE_BYTES // 4, dtype=torch.int32, device=device)
        _pools[(idx, st)] = pool
    return pool, st


def workspace(device: torch.device) -> torch.Tensor:
    return workspace_and_stream(device)[0]


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def update_scaling_factor_host(amax: float, old: float, fmt: int, margin: int) -> float:
    return float(_lib.ntfp8_update_scaling_factor_host(amax, old, fmt, margin))
