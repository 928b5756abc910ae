import torch

from nanotron_amd.fp8.constants import FP8_GPU_NAMES


def is_fp8_available() -> bool:
    """True when the current device is a CDNA4 part (reference: src/nanotron/fp8/utils.py:7-13,
    same substring test against its own list of device names)."""
    if not torch.cuda.is_available():
        return False
    idx = torch.cuda.current_device()
    name = torch.cuda.get_device_name(idx).lower()
    arch = getattr(torch.cuda.get_device_properties(idx), "gcnArchName", "").lower()
    return any(g in name or g in arch for g in FP8_GPU_NAMES)
