import torch
from torch import nn

from nanotron_amd.fp8.constants import FP8_DTYPES
from nanotron_amd.fp8.dtypes import DTypes
from nanotron_amd.fp8.meta import FP8Meta
from nanotron_amd.fp8.tensor import FP8Tensor


def _quantised(hp: torch.Tensor, dtype: DTypes) -> FP8Tensor:
    """The fp8 copy of a high-precision weight.  The dgrad GEMM reduces over the weight's rows: the copy carries its
    transpose unless the library reads the weight as it is (`ntfp8_gemm_desc.b_transposed`)."""
    from nanotron_amd.fp8.kernel import needs_transposed_copy

    return FP8Tensor(hp, dtype=dtype, with_transpose=hp.dim() == 2 and needs_transposed_copy(hp.shape[0], hp.shape[1]))


def _checked(source) -> torch.Tensor:
    # the reference's three preconditions, with its messages (src/nanotron/fp8/parameter.py:17-20)
    assert isinstance(source, torch.Tensor), "data must be a tensor"
    assert source.dtype not in FP8_DTYPES, "Currently only support turn a non-fp8 tensor to an fp8 parameter"
    assert source.device != torch.device("cpu"), "FP8Parameter only supports CUDA tensors"
    return source


class FP8Parameter(nn.Parameter):
    """Parameter whose own storage stays high precision (so autograd and optimizers accept it) and
    whose `.data` is the quantised FP8Tensor (reference: src/nanotron/fp8/parameter.py:10-43)."""

    def __new__(cls, data: torch.Tensor, dtype: DTypes, requires_grad: bool = True) -> nn.Parameter:
        hp = _checked(data)
        with torch.no_grad():
            param = torch.Tensor._make_subclass(cls, hp, requires_grad)
            param._fp8_dtype = dtype
            param._data = _quantised(hp, dtype)
        return param

    @property
    def data(self) -> FP8Tensor:
        return self._data

    @data.setter
    def data(self, data: FP8Tensor):
        self._data = data

    @property
    def fp8_meta(self) -> FP8Meta:
        return self.data.fp8_meta

    @torch.no_grad()
    def requantize(self) -> None:
        """Refresh the fp8 copy (and its transpose, where one is kept) from the high-precision storage, e.g. after an
        optimizer step.  The reference never does this (parameter.py:27 runs once)."""
        self._data = _quantised(self.as_subclass(torch.Tensor), self._fp8_dtype)

    def __repr__(self) -> str:
        return f"FP8Parameter({self.data!r}, requires_grad={self.requires_grad})"
