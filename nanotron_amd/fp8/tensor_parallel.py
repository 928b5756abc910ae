"""FP8 column- and row-parallel linears for a tensor-parallel group of one GPU.

The reference's tensor-parallel linears (src/nanotron/parallel/tensor_parallel/nn.py:46-176) are
`nn.Linear` subclasses whose forward is `column_linear` / `row_linear`
(src/nanotron/parallel/tensor_parallel/functional.py:548-567, 704-725): an `F.linear` between
differentiable collectives that are identities when the group has one rank
(distributed_differentiable_primitives.py:43,61,99).  The classes here keep those constructors and
replace the `F.linear` with the FP8 path of `FP8Linear`, so the projections of a LLaMA block
(src/nanotron/models/llama.py:227-246, 388-432) run on the fp8 matrix cores.

Only a group of one rank is served: with one GPU per process and one GPU in the machine there is
nothing to exchange, and a larger group raises instead of computing a partial result.
"""
from enum import Enum, auto
from typing import Optional, Tuple

import torch

from nanotron_amd.fp8.linear import FP8Linear


class TensorParallelLinearMode(Enum):
    """src/nanotron/parallel/tensor_parallel/enum.py:4-12."""

    ALL_REDUCE = auto()
    REDUCE_SCATTER = auto()

    def __format__(self, format_spec):
        return self.name

    def __str__(self):
        return self.name


def _group_size(pg) -> int:
    """Ranks in `pg`; None stands for a process that never initialised torch.distributed."""
    return 1 if pg is None else pg.size()


def _group_rank(pg) -> int:
    """This process's rank in `pg` (dist.get_rank(pg) in the reference): the only rank of a one-rank group."""
    if _group_size(pg) == 1:
        return 0
    import torch.distributed as dist

    return dist.get_rank(pg)


def _require_single_rank(pg, what: str) -> None:
    n = _group_size(pg)
    if n != 1:
        raise NotImplementedError(
            f"{what}: tensor-parallel group of {n} ranks; this build serves one GPU and exchanges no shards "
            "(a column-parallel layer would all-reduce / reduce-scatter dX, a row-parallel layer Y, and every "
            "quantised tensor's amax would be max-reduced over the group before its scale is taken)")


class FP8TensorParallelColumnLinear(FP8Linear):
    """Output features split over the group (nn.py:46-110).  Constructor as the reference's, plus
    FP8Linear's keyword-only extensions."""

    def __init__(self, in_features, out_features, pg, mode: TensorParallelLinearMode, bias=True, device=None,
                 dtype=None, async_communication: bool = False, contiguous_chunks: Optional[Tuple[int, ...]] = None,
                 tp_recompute_allgather: bool = True, **fp8_kwargs):
        _require_single_rank(pg, type(self).__name__)
        if not isinstance(mode, TensorParallelLinearMode):
            raise ValueError(f"Got unexpected mode: {mode}.")
        self.pg = pg
        self.world_size = _group_size(pg)
        assert out_features % self.world_size == 0
        if contiguous_chunks is not None:
            assert (
                sum(contiguous_chunks) == out_features
            ), f"Sum of contiguous chunks ({sum(contiguous_chunks)}) must equal to out_features ({out_features})"
        super().__init__(in_features, out_features // self.world_size, bias, device, dtype=dtype, **fp8_kwargs)
        self.mode = mode
        self.async_communication = async_communication
        self.tp_recompute_allgather = tp_recompute_allgather
        self.contiguous_chunks = contiguous_chunks

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        # both modes, synchronous or not: identity / all-gather of one rank, then the linear (functional.py:557-566)
        return super().forward(x)

    def extra_repr(self) -> str:
        return (f"tp_rank={_group_rank(self.pg)}, {super().extra_repr()}, "
                f"unsharded_out_features={self.out_features * self.world_size}")


class FP8TensorParallelRowLinear(FP8Linear):
    """Input features split over the group (nn.py:113-176)."""

    def __init__(self, in_features, out_features, pg, mode: TensorParallelLinearMode, bias=True, device=None,
                 dtype=None, async_communication: bool = False, contiguous_chunks: Optional[Tuple[int, ...]] = None,
                 **fp8_kwargs):
        _require_single_rank(pg, type(self).__name__)
        if not isinstance(mode, TensorParallelLinearMode):
            raise ValueError(f"Got unexpected mode: {mode}.")
        if mode is TensorParallelLinearMode.ALL_REDUCE and async_communication:
            raise ValueError("async_communication is not supported for ALL_REDUCE mode")
        self.pg = pg
        self.world_size = _group_size(pg)
        assert in_features % self.world_size == 0
        if contiguous_chunks is not None:
            assert (
                sum(contiguous_chunks) == in_features
            ), f"Sum of contiguous chunks ({sum(contiguous_chunks)}) must equal to in_features ({in_features})"
        # only rank 0 of the group keeps the bias (nn.py:135-136)
        bias = _group_rank(pg) == 0 and bias
        super().__init__(in_features // self.world_size, out_features, bias, device, dtype=dtype, **fp8_kwargs)
        self.mode = mode
        self.async_communication = async_communication
        self.contiguous_chunks = contiguous_chunks

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        # the linear, then an all-reduce / reduce-scatter of one rank (functional.py:715-725)
        return super().forward(x)

    def extra_repr(self) -> str:
        return (f"tp_rank={_group_rank(self.pg)}, {super().extra_repr()}, "
                f"unsharded_in_features={self.in_features * self.world_size}")
