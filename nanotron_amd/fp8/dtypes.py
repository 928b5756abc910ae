"""Format tags, same names and values as the reference (src/nanotron/fp8/dtypes.py:4-7), plus the
stand-in for Transformer Engine's `tex.DType` enum that `FP8Meta.te_dtype` returns."""
from enum import Enum, IntEnum, auto


class DTypes(Enum):
    FP8E4M3 = auto()
    FP8E5M2 = auto()
    KFLOAT16 = auto()


class DType(IntEnum):
    """Element types understood by the native library; member names follow tex.DType
    (used at src/nanotron/fp8/tensor.py:39-55)."""

    kByte = 0
    kInt32 = 1
    kFloat32 = 2
    kFloat16 = 3
    kBFloat16 = 4
    kFloat8E4M3 = 5
    kFloat8E5M2 = 6
