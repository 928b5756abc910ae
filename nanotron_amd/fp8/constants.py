"""Constants of the FP8 path (reference: src/nanotron/fp8/constants.py:5-18)."""
import torch

from nanotron_amd.fp8.dtypes import DTypes

# Device-name substrings on which the FP8 kernels run.  The reference lists NVIDIA parts
# ("h100", "rtx 4090"); this implementation targets CDNA4.
FP8_GPU_NAMES = ["mi355", "mi350", "gfx950"]

INITIAL_AMAX = 1.0
INITIAL_SCALING_FACTOR = 1.0

# Storage dtypes that mark a tensor as already quantised.  Bytes are stored as uint8 for both
# formats (tests/fp8/test_tensor.py:23); the two names below are kept for import compatibility.
FP8_DTYPES = [torch.int8, torch.uint8]
FP8E4M3_DTYPE = torch.int8
FP8E5M2_DTYPE = torch.uint8

DTYPE_TO_FP8_MAX = {DTypes.FP8E4M3: 448.0, DTypes.FP8E5M2: 57344.0, DTypes.KFLOAT16: 65504.0}

# Delayed-scaling defaults of the benchmark configurations (not in the reference).
DEFAULT_AMAX_HISTORY_LEN = 16
DEFAULT_MARGIN = 0
