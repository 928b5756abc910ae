import torch
from torch import nn

from nanotron_amd.fp8.constants import FP8_DTYPES
from nanotron_amd.fp8.dtypes import DTypes
from nanotron_amd.fp8.meta import FP8Meta
from nanotron_amd.fp8.tensor import FP8Tensor


def _with_transpose(w: torch.Tensor) -> bool:
    """The dgrad GEMM reduces over the weight's rows: it gets a transposed copy unless the library reads it as it is."""
    from nanotron_amd.fp8.kernel import needs_transposed_copy

    return w.dim() == 2 and needs_transposed_copy(w.shape[0], w.shape[1])


class FP8Parameter(nn.Parameter):
    """Parameter whose own storage stays high precision (so autograd and optimizers accept it) and
    whose `.data` is the quantised FP8Tensor (reference: src/nanotron/fp8/parameter.py:10-43).

    The quantised copy is produced together with its transpose, which the dgrad GEMM consumes, unless the
    library's GEMM can read the weight as it is (`ntfp8_gemm_desc.b_transposed`)."""

    def __new__(cls, data: torch.Tensor, dtype: DTypes, requires_grad: bool = True) -> nn.Parameter:
        assert isinstance(data, torch.Tensor), "data must be a tensor"
        assert data.dtype not in FP8_DTYPES, "Currently only support turn a non-fp8 tensor to an fp8 parameter"
        assert data.device != torch.device("cpu"), "FP8Parameter only supports CUDA tensors"

        with torch.no_grad():
            self = torch.Tensor._make_subclass(cls, data, requires_grad)
            self._fp8_dtype = dtype
            self._data = FP8Tensor(data, dtype=dtype, with_transpose=_with_transpose(data))
        return self

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
        """Refresh the fp8 copy (and its transpose) from the high-precision storage, e.g. after an
        optimizer step.  The reference never does this (parameter.py:27 runs once)."""
        hp = self.as_subclass(torch.Tensor)
        self._data = FP8Tensor(hp, dtype=self._fp8_dtype, with_transpose=_with_transpose(hp))

    def __repr__(self) -> str:
        return f"FP8Parameter({self.data!r}, requires_grad={self.requires_grad})"
