"""Keeping the fp8 weight copies in step with their high-precision masters.

The reference quantises a weight once, when the FP8Parameter is built (src/nanotron/fp8/parameter.py:27),
and never again; its optimizers update the high-precision storage only
(src/nanotron/optim/gradient_accumulator.py:257-267 copies the fp32 master back into the half-precision
parameter after each step).  A training loop therefore has to refresh the fp8 copy, and the transposed copy the
dgrad GEMM reads, after every optimizer step; these helpers do that."""
from typing import Iterable, Optional, Union

import torch
from torch import nn

from nanotron_amd.fp8.linear import FP8Linear


def fp8_linears(module_or_modules: Union[nn.Module, Iterable[nn.Module]]):
    """Every FP8Linear reachable from the argument (a module, or an iterable of modules)."""
    mods = [module_or_modules] if isinstance(module_or_modules, nn.Module) else list(module_or_modules)
    seen = set()
    for root in mods:
        for m in root.modules():
            if isinstance(m, FP8Linear) and id(m) not in seen:
                seen.add(id(m))
                yield m


@torch.no_grad()
def requantize_fp8_weights(module_or_modules, stream: Optional[torch.cuda.Stream] = None) -> int:
    """Re-quantise the weight of every FP8Linear from its master copy (one delayed-scaling step for the
    weight role where delayed scaling is on).  Returns the number of layers refreshed."""
    n = 0
    for lin in fp8_linears(module_or_modules):
        if lin.weight.device.type == "cpu":
            continue
        lin.requantize_weight(stream=stream)
        n += 1
    return n


def attach_requantize_hook(optimizer: torch.optim.Optimizer, module_or_modules, stream: Optional[torch.cuda.Stream] = None):
    """After every `optimizer.step()` refresh the fp8 weights of the given modules.  Returns the hook handle
    (`.remove()` detaches it)."""
    layers = list(fp8_linears(module_or_modules))

    def _hook(opt, args, kwargs):
        requantize_fp8_weights(layers, stream=stream)

    return optimizer.register_step_post_hook(_hook)
