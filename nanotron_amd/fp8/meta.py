from dataclasses import dataclass
from typing import Union

import torch

from nanotron_amd.fp8.constants import DTYPE_TO_FP8_MAX
from nanotron_amd.fp8.dtypes import DType, DTypes


@dataclass
class FP8Meta:
    """Metadata of an FP8Tensor (reference: src/nanotron/fp8/meta.py:12-40): field order
    (amax, scale, dtype) and the three properties are the reference's."""

    amax: Union[int, float, torch.Tensor]
    scale: torch.Tensor
    dtype: DTypes

    @property
    def te_dtype(self) -> DType:
        from nanotron_amd.fp8.tensor import convert_torch_dtype_to_te_dtype

        return convert_torch_dtype_to_te_dtype(self.dtype)

    def __post_init__(self):
        if not isinstance(self.amax, torch.Tensor):
            if isinstance(self.scale, torch.Tensor) and self.scale.is_cuda:
                device = self.scale.device
            else:
                device = "cuda" if torch.cuda.is_available() else "cpu"
            self.amax = torch.tensor(self.amax, device=device)

    @property
    def fp8_max(self) -> float:
        return DTYPE_TO_FP8_MAX[self.dtype]

    @property
    def inverse_scale(self) -> torch.Tensor:
        return 1 / self.scale

    def __repr__(self) -> str:
        return f"FP8Meta(amax={self.amax}, scale={self.scale}, inverse_scale={self.inverse_scale}, dtype={self.dtype})"
