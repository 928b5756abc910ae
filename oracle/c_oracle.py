"""ctypes binding of oracle/libfp8oracle.so (the C restatement).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libfp8oracle.so")

FMT = {"e4m3": 0, "e5m2": 1}
DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def build() -> str:
    subprocess.check_call(["make", "-s", "-C", _HERE, "libfp8oracle.so"])
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        c = ctypes
        L.orc_amax.restype = c.c_float
        L.orc_amax.argtypes = [c.c_void_p, c.c_int, c.c_int64]
        L.orc_update_scale.restype = c.c_float
        L.orc_update_scale.argtypes = [c.c_float, c.c_float, c.c_int, c.c_int]
        L.orc_encode_fp8.restype = c.c_uint8
        L.orc_encode_fp8.argtypes = [c.c_float, c.c_int]
        L.orc_decode_fp8.restype = c.c_float
        L.orc_decode_fp8.argtypes = [c.c_uint8, c.c_int]
        L.orc_cast_to_fp8.restype = None
        L.orc_cast_to_fp8.argtypes = [c.c_void_p, c.c_int, c.c_int64, c.c_float, c.c_int, c.c_void_p]
        L.orc_cast_from_fp8.restype = None
        L.orc_cast_from_fp8.argtypes = [c.c_void_p, c.c_int64, c.c_float, c.c_int, c.c_void_p]
        L.orc_transpose.restype = None
        L.orc_transpose.argtypes = [c.c_void_p, c.c_int64, c.c_int64, c.c_void_p]
        L.orc_gemm_nt.restype = None
        L.orc_gemm_nt.argtypes = [c.c_void_p, c.c_int, c.c_float, c.c_void_p, c.c_int, c.c_float,
                                  c.c_void_p, c.c_int64, c.c_int64, c.c_int64, c.c_int]
        L.orc_delayed_step.restype = c.c_float
        L.orc_delayed_step.argtypes = [c.c_void_p, c.c_int, c.c_int64, c.c_int, c.c_int, c.c_void_p, c.c_int,
                                       c.c_void_p, c.c_void_p, c.c_void_p, c.c_void_p]
        _lib = L
    return _lib


def amax(x: torch.Tensor) -> float:
    x = x.contiguous()
    return float(lib().orc_amax(x.data_ptr(), DT[x.dtype], x.numel()))


def update_scale(amax_: float, old: float, fmt: str, margin: int = 0) -> float:
    return float(lib().orc_update_scale(amax_, old, FMT[fmt], int(margin)))


def cast_to_fp8(x: torch.Tensor, scale: float, fmt: str) -> torch.Tensor:
    x = x.contiguous()
    out = torch.empty(x.shape, dtype=torch.uint8)
    lib().orc_cast_to_fp8(x.data_ptr(), DT[x.dtype], x.numel(), scale, FMT[fmt], out.data_ptr())
    return out


def cast_from_fp8(q: torch.Tensor, scale: float, fmt: str) -> torch.Tensor:
    q = q.contiguous()
    out = torch.empty(q.shape, dtype=torch.float32)
    lib().orc_cast_from_fp8(q.data_ptr(), q.numel(), scale, FMT[fmt], out.data_ptr())
    return out


def decode_table(fmt: str) -> np.ndarray:
    return np.array([lib().orc_decode_fp8(b, FMT[fmt]) for b in range(256)], dtype=np.float32)


def transpose(q: torch.Tensor) -> torch.Tensor:
    q = q.contiguous()
    out = torch.empty((q.shape[1], q.shape[0]), dtype=torch.uint8)
    lib().orc_transpose(q.data_ptr(), q.shape[0], q.shape[1], out.data_ptr())
    return out


def gemm_nt(a, fmt_a, scale_a, b, fmt_b, scale_b, accumulate_into=None) -> torch.Tensor:
    a = a.contiguous()
    b = b.contiguous()
    M, K = a.shape
    N, K2 = b.shape
    assert K == K2
    d = accumulate_into.clone().contiguous() if accumulate_into is not None else torch.empty((M, N), dtype=torch.float32)
    lib().orc_gemm_nt(a.data_ptr(), FMT[fmt_a], scale_a, b.data_ptr(), FMT[fmt_b], scale_b,
                      d.data_ptr(), M, N, K, 1 if accumulate_into is not None else 0)
    return d


class DelayedScalingC:
    def __init__(self, fmt: str, history_len: int = 16, margin: int = 0):
        self.fmt, self.H, self.margin = fmt, history_len, margin
        self.hist = torch.zeros(history_len, dtype=torch.float32)
        self.scale = ctypes.c_float(1.0)
        self.init = ctypes.c_int(0)

    def quantise(self, x: torch.Tensor):
        x = x.contiguous()
        out = torch.empty(x.shape, dtype=torch.uint8)
        used = ctypes.c_float(0)
        a = lib().orc_delayed_step(x.data_ptr(), DT[x.dtype], x.numel(), FMT[self.fmt], self.margin,
                                   self.hist.data_ptr(), self.H, ctypes.byref(self.scale), ctypes.byref(self.init),
                                   out.data_ptr(), ctypes.byref(used))
        return out, float(a), float(used.value)
