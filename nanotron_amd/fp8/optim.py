"""Keeping the fp8 weight copies in step with their high-precision masters.

The reference quantises a weight once, when the FP8Parameter is built (src/nanotron/fp8/parameter.py:27),
and never again; its optimizers update the high-precision storage only
(src/nanotron/optim/gradient_accumulator.py:257-267 copies the fp32 master back into the half-precision
parameter after each step).  A training loop therefore has to refresh the fp8 copy, and the transposed copy the
dgrad GEMM reads, after every optimizer step; these helpers do that."""
from typing import Iterable, Optional, Union

import torch
from torch import nn

from nanotron_amd.fp8.dtypes import DTypes
from nanotron_amd.fp8.kernel import needs_transposed_copy
from nanotron_amd.fp8.linear import FP8Linear
from nanotron_amd.fp8.tensor import quantize_delayed_batch


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
    layers = [lin for lin in fp8_linears(module_or_modules) if lin.weight.device.type != "cpu"]
    rest = layers
    if stream is None:
        # weights whose delayed-scaling role already holds a scale go through one batched library call per device
        ready = [lin for lin in layers if lin.scaling is not None and lin.scaling["weight"].known_initialised]
        by_device = {}
        for lin in ready:
            by_device.setdefault(lin.weight.device, []).append(lin)
        batched = set()
        for dev, lins in by_device.items():
            if len(lins) < 2:
                continue
            with torch.cuda.device(dev):
                hp = [lin.weight.as_subclass(torch.Tensor) for lin in lins]
                qs = quantize_delayed_batch(hp, DTypes.FP8E4M3, [lin.scaling["weight"] for lin in lins],
                                            [needs_transposed_copy(*w.shape) for w in hp])
            for lin, q in zip(lins, qs):
                lin.weight.data = q
                lin._weight_ready = None
                batched.add(id(lin))
        rest = [lin for lin in layers if id(lin) not in batched]
    for lin in rest:
        lin.requantize_weight(stream=stream)
    return len(layers)


def attach_requantize_hook(optimizer: torch.optim.Optimizer, module_or_modules, stream: Optional[torch.cuda.Stream] = None):
    """After every `optimizer.step()` refresh the fp8 weights of the given modules.  Returns the hook handle
    (`.remove()` detaches it)."""
    layers = list(fp8_linears(module_or_modules))

    def _hook(opt, args, kwargs):
        requantize_fp8_weights(layers, stream=stream)

    return optimizer.register_step_post_hook(_hook)
