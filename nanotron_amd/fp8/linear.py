from typing import Optional, Tuple, TypedDict, Union

import torch
import torch.nn.functional as F
from torch import nn

from nanotron_amd.fp8.constants import INITIAL_AMAX, INITIAL_SCALING_FACTOR
from nanotron_amd.fp8.dtypes import DTypes
from nanotron_amd.fp8.kernel import a_transposed_supported, fp8_matmul_kernel, fp8_matmul_pair, needs_transposed_copy
from nanotron_amd.fp8.meta import FP8Meta
from nanotron_amd.fp8.parameter import FP8Parameter
from nanotron_amd.fp8.tensor import DelayedScaling, FP8Tensor, cast_with_scale, update_scaling_factor


class FP8LinearMeta(TypedDict):
    """FP8 metadata for FP8Linear (reference: src/nanotron/fp8/linear.py:16-21)."""

    input_grad: FP8Meta
    weight_grad: FP8Meta
    output_grad: FP8Meta


class _GradBox:
    """What travels beside the autograd graph between an FP8Linear with an fp8 output and the layer that consumes it:
    the delayed-scaling role the producer quantises its output gradient with, and, during a backward pass, that
    gradient already as e5m2 bytes out of the consumer's dgrad epilogue (autograd itself only carries a placeholder
    then: a gradient must have its tensor's type, and the tensor it stands for is the high-precision handle).
    `consumers` counts the layers whose forward took the activation with gradients on: fp8 contributions cannot be
    summed, so the fp8 hand-over is used only while there is exactly one, and an activation with several consumers
    gets high-precision gradients that autograd sums."""

    __slots__ = ("state", "fp8_grad", "arrivals", "consumers")

    def __init__(self, state):
        self.state, self.fp8_grad, self.arrivals, self.consumers = state, None, 0, 0


class FP8Linear(nn.Linear):
    """nn.Linear whose matmuls run in FP8 (reference: src/nanotron/fp8/linear.py:24-66).

    Positional signature as the reference.  Keyword-only extensions, all defaulting to the
    reference's behaviour: `dtype` (of the master weight and bias, as nn.Linear's), `out_dtype`
    (None = fp32 output, kernel.py:24,28; `DTypes.FP8E4M3` / `FP8E5M2` = the output is returned as an
    FP8Tensor, the TODO at linear.py:63-64, quantised in the GEMM epilogue with the delayed-scaling role "output",
    its transposed copy included if `fp8_output_transpose`; it carries a gradient handle, so that a following
    FP8Linear back-propagates into this one, see _FP8Matmul), `delayed_scaling`
    (False = scale every tensor from its own amax), `amax_history_len`, `margin`,
    `accumulate_grad` (False = `weight.grad` is overwritten each backward, linear.py:110; True =
    the wgrad GEMM adds into the existing fp32 gradient in its epilogue).  With a bf16 / fp16
    master weight the fp32 weight gradient is stored as `weight.main_grad` instead of `.grad`.
    The bias is added inside the GEMM epilogue (the TODO at linear.py:62).  In evaluation mode (`module.eval()`)
    tensors are quantised with the scales the delayed-scaling roles hold and the roles are left untouched."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, device: Optional[torch.device] = None,
                 *, dtype: Optional[torch.dtype] = None, out_dtype: Union[torch.dtype, DTypes, None] = None,
                 delayed_scaling: bool = False, amax_history_len: int = 16, margin: int = 0,
                 accumulate_grad: bool = False, fp8_output_transpose: bool = False):
        super().__init__(in_features, out_features, bias, device, dtype)
        if isinstance(out_dtype, DTypes):
            if out_dtype not in (DTypes.FP8E4M3, DTypes.FP8E5M2):
                raise ValueError(f"{out_dtype} is not an FP8 format")
        self.out_dtype = out_dtype
        self.fp8_output_transpose = fp8_output_transpose
        self.accumulate_grad = accumulate_grad
        # True: every backward leaves the quantised output gradient (the FP8Tensor both backward GEMMs read) in
        # `self.quantised_grad_output`, as autograd keeps the quantised input in `saved_tensors`; off by default, the
        # reference drops it (linear.py:102) and it would pin the bytes until the next backward
        self.keep_quantised_grad = False
        self.quantised_grad_output = None
        # True: the gradient of an fp8 input that another FP8Linear produced goes back to that layer as e5m2 bytes
        # straight from this layer's dgrad epilogue (cast with the producer's output-gradient scale) instead of as a
        # high-precision tensor the producer then quantises; the producer's bias gradient is then summed from the
        # e5m2 values.  Used only while this layer is the activation's one consumer
        self.fp8_grad_input = True
        self.fp8_grad_inputs_sent = 0   # backward passes of this layer that did so
        self._grad_box = None
        self.scaling = None
        self._weight_ready = None
        if self.weight.device != torch.device("cpu"):
            self.weight = FP8Parameter(self.weight, dtype=DTypes.FP8E4M3)

            # quantisation metadata for input / weight / output gradients, as linear.py:33-49
            fp8e4m3_scale = update_scaling_factor(
                amax=torch.tensor(INITIAL_AMAX, dtype=torch.float32),
                scaling_factor=torch.tensor(INITIAL_SCALING_FACTOR, dtype=torch.float32),
                dtype=DTypes.FP8E4M3,
            )
            fp8e5m2_scale = update_scaling_factor(
                amax=torch.tensor(INITIAL_AMAX, dtype=torch.float32),
                scaling_factor=torch.tensor(INITIAL_SCALING_FACTOR, dtype=torch.float32),
                dtype=DTypes.FP8E5M2,
            )
            self.fp8_meta: FP8LinearMeta = {
                "input_grad": FP8Meta(amax=1, dtype=DTypes.FP8E4M3, scale=fp8e4m3_scale),
                "weight_grad": FP8Meta(amax=1, dtype=DTypes.FP8E4M3, scale=fp8e4m3_scale),
                "output_grad": FP8Meta(amax=1, dtype=DTypes.FP8E5M2, scale=fp8e5m2_scale),
            }
            if delayed_scaling:
                dev = self.weight.device
                self.scaling = {
                    "input": DelayedScaling(DTypes.FP8E4M3, amax_history_len, margin, dev),
                    "weight": DelayedScaling(DTypes.FP8E4M3, amax_history_len, margin, dev),
                    "output_grad": DelayedScaling(DTypes.FP8E5M2, amax_history_len, margin, dev),
                }
                if isinstance(out_dtype, DTypes):
                    self.scaling["output"] = DelayedScaling(out_dtype, amax_history_len, margin, dev)

    @torch.no_grad()
    def requantize_weight(self, stream: Optional[torch.cuda.Stream] = None) -> None:
        """Refresh the fp8 weight (and its transpose) from the high-precision master copy; with
        delayed scaling this advances the weight role's amax history by one step.

        With `stream`, the (HBM-bound) quantisation is queued on that stream behind the work already
        on the current one, so it overlaps whatever the current stream does next (typically the
        MFMA-bound GEMMs of other layers); the next forward of this layer waits for it."""
        w = self.weight
        hp = w.as_subclass(torch.Tensor)
        state = self.scaling["weight"] if self.scaling is not None else None
        if stream is None:
            w.data = FP8Tensor(hp, dtype=DTypes.FP8E4M3, state=state, with_transpose=needs_transposed_copy(*hp.shape))
            self._weight_ready = None
            return
        cur = torch.cuda.current_stream(hp.device)
        stream.wait_stream(cur)
        with torch.cuda.stream(stream):
            q = FP8Tensor(hp, dtype=DTypes.FP8E4M3, state=state, with_transpose=needs_transposed_copy(*hp.shape))
            ready = torch.cuda.Event()
            ready.record(stream)
        # the new tensors were allocated on `stream` and will be read on the current one
        for t in (q, getattr(q, "_transposed", None), q.fp8_meta.amax):
            if t is None:
                continue
            t.record_stream(cur)
        w.data = q
        self._weight_ready = ready

    # ---- checkpoints -------------------------------------------------------------------------------
    # The reference serialises no FP8 state (nothing under src/nanotron/serialize knows about it).  Here a
    # layer with delayed scaling adds four fp32 tensors to its state dict, `fp8_state.<role>` =
    # [seen a usable amax (0/1), scale for the next step, amax history newest first] and
    # `fp8_state.weight_scale` = the scale the current fp8 weight copy was cast with, so that a resumed run
    # continues the delayed-scaling trajectory bit for bit.  Layers without delayed scaling add nothing, and
    # a state dict without these keys loads as before.
    _FP8_STATE = "fp8_state."

    def _save_to_state_dict(self, destination, prefix, keep_vars):
        super()._save_to_state_dict(destination, prefix, keep_vars)
        if self.scaling is None:
            return
        for role, st in self.scaling.items():
            flag = torch.tensor([1.0 if st.initialised else 0.0], dtype=torch.float32, device=st._buf.device)
            destination[prefix + self._FP8_STATE + role] = torch.cat([flag, st._buf.detach()])
        destination[prefix + self._FP8_STATE + "weight_scale"] = self.weight.fp8_meta.scale.detach().reshape(1).clone()

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs):
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs)
        mine = {k: v for k, v in state_dict.items() if k.startswith(prefix + self._FP8_STATE)}
        for k in mine:
            if k in unexpected_keys:
                unexpected_keys.remove(k)
        if not isinstance(self.weight, FP8Parameter):
            return
        weight_scale = None
        if self.scaling is not None:
            for role, st in self.scaling.items():
                t = mine.get(prefix + self._FP8_STATE + role)
                if t is None:
                    if strict:
                        missing_keys.append(prefix + self._FP8_STATE + role)
                    continue
                if t.numel() != 2 + st.history_len:
                    error_msgs.append(f"{prefix}{self._FP8_STATE}{role}: amax history of length {t.numel() - 2}, "
                                      f"this layer keeps {st.history_len}")
                    continue
                t = t.to(device=st._buf.device, dtype=torch.float32)
                st._buf.copy_(t[1:])
                st.initialised = bool(t[0].item() != 0.0)
            weight_scale = mine.get(prefix + self._FP8_STATE + "weight_scale")
        # the master weight has just been overwritten: rebuild the fp8 copy (and its transpose) from it
        w = self.weight
        hp = w.as_subclass(torch.Tensor)
        with torch.no_grad():
            if weight_scale is not None:
                w.data = cast_with_scale(hp, weight_scale, DTypes.FP8E4M3, with_transpose=needs_transposed_copy(*hp.shape))
            else:
                w.data = FP8Tensor(hp, dtype=DTypes.FP8E4M3, with_transpose=needs_transposed_copy(*hp.shape))
        self._weight_ready = None

    def forward(self, input: Union[FP8Tensor, torch.Tensor]) -> torch.Tensor:
        # fp8 kernels only when both input and weight are on the GPU (linear.py:53-54)
        if input.device == torch.device("cpu") or self.weight.device == torch.device("cpu"):
            return F.linear(input, self.weight, self.bias)

        if self._weight_ready is not None:  # weight re-quantisation queued on another stream
            torch.cuda.current_stream(input.device).wait_event(self._weight_ready)
            self._weight_ready = None

        # phony tensor that makes autograd call our backward although the weight's gradient is
        # produced by the fp8 kernels, not by autograd (linear.py:56-60)
        phony = torch.empty(0, device=input.device, requires_grad=True)
        # The bias goes into the GEMM's epilogue (the TODO at linear.py:62; for the fp32 output of the reference the
        # result equals `output + self.bias`, linear.py:65, bit for bit) and an fp8 input produced by another
        # FP8Linear brings the handle its gradient travels through (below).
        handle = getattr(input, "_grad_handle", None)
        if handle is None and torch.is_grad_enabled() and getattr(getattr(input, "fp8_meta", None), "from_fp8_linear", False):
            # the bytes of another FP8Linear's output, but not the object it returned (a view, a copy or a slice with
            # the meta carried over): the producer would silently get no gradient
            raise RuntimeError("this fp8 activation was produced by an FP8Linear but has lost the gradient handle that "
                               "layer attached to its output (`_grad_handle`): pass the output object itself, or carry "
                               "the attribute over to the tensor derived from it")
        if handle is not None and handle.requires_grad and torch.is_grad_enabled():
            box = getattr(handle, "_grad_box", None)
            if box is not None:
                box.consumers += 1
        output, aux = _FP8Matmul.apply(input, self.weight, self.fp8_meta, phony, self, self.bias, handle)
        if isinstance(self.out_dtype, DTypes):
            output._grad_handle = aux
            aux._grad_box = self._grad_box   # made by this forward: where a consuming layer leaves an fp8 gradient
            output.fp8_meta.from_fp8_linear = True   # travels with the meta if a caller re-wraps the bytes
        return output


class _FP8Matmul(torch.autograd.Function):
    """Y = X.W^T forward; dX = dY.W and dW = dY^T.X backward, all three on the fp8 matrix cores
    (reference: src/nanotron/fp8/linear.py:69-112).  The backward computes the gradients its
    docstring states (linear.py:92-96) for any shape and uses the real upstream gradient.

    `apply(input, weight, fp8_meta, phony)` is the reference's call (linear.py:60): current scaling, fp32 output.
    Three more positional arguments carry this build's extensions: `module` (the FP8Linear: output type, delayed
    scaling roles, gradient accumulation), `bias` (added in the GEMM epilogue; its gradient is returned like any
    other) and `input_handle`.

    fp8 activations and autograd.  With `module.out_dtype` an FP8 format the output is an FP8Tensor, a uint8 tensor
    that cannot carry a gradient.  The second output then is its *gradient handle*: a [tokens, out_features] tensor
    of the high-precision type without memory of its own (one element, expanded), part of the autograd graph.  The
    FP8Linear that consumes the FP8Tensor passes the handle along as `input_handle`; its backward returns dX as the
    handle's gradient, and autograd delivers it to the producer's backward as the gradient of the output it stands
    for.  So a chain FP8Linear(out_dtype=E4M3) -> FP8Linear trains without the activation ever leaving fp8."""

    @staticmethod
    @torch.no_grad()
    def forward(ctx, input, weight, fp8_meta, phony: torch.Tensor, module: Optional["FP8Linear"] = None,
                bias: Optional[torch.Tensor] = None, input_handle: Optional[torch.Tensor] = None):
        scaling = module.scaling if module is not None else None
        update = module.training if module is not None else True   # evaluation passes leave the scaling state alone
        needs_wgrad = weight.requires_grad
        ctx.in_dtype = input.dtype if type(input) == torch.Tensor else (input_handle.dtype if input_handle is not None else None)
        ctx.in_shape = input.shape
        ctx.has_handle = input_handle is not None
        ctx.input_box = getattr(input_handle, "_grad_box", None) if input_handle is not None else None
        if type(input) == torch.Tensor:
            x2d = input.reshape(-1, input.shape[-1])
            input = FP8Tensor(x2d, dtype=DTypes.FP8E4M3, state=scaling["input"] if scaling else None,
                              with_transpose=needs_wgrad and needs_transposed_copy(x2d.shape[0], x2d.shape[1], weight.shape[0]),
                              update_state=update)
        ctx.save_for_backward(input, weight, bias)
        ctx.module = module
        ctx.fp8_meta = fp8_meta
        out_dtype = (module.out_dtype if module is not None else None) or torch.float32
        gemm_bias = bias.detach() if bias is not None else None

        # FP8Tensor of the weight, not the FP8Parameter (linear.py:81-84)
        if isinstance(out_dtype, DTypes):
            # [tokens, out_features] whatever the input's leading dimensions: what the next layer's GEMM consumes
            state = scaling["output"] if scaling else None
            if state is not None and not update and state.initialised:
                state = _frozen_copy(state)
            output = fp8_matmul_kernel(
                mat_a=weight.data, transpose_a=True, mat_b=input, transpose_b=False, use_split_accumulator=False,
                out_dtype=out_dtype, out_state=state, out_with_transpose=module.fp8_output_transpose, bias=gemm_bias,
            )
            ctx.mark_non_differentiable(output)
            ctx.grad_box = module._grad_box = _GradBox(scaling["output_grad"] if scaling else None)
            hp = weight.dtype if weight.dtype in (torch.float32, torch.float16, torch.bfloat16) else torch.float32
            handle = torch.zeros(1, dtype=hp, device=output.device).expand(output.shape)
            ctx.fp8_out = True
            return output, handle
        ctx.fp8_out = False
        output = fp8_matmul_kernel(
            mat_a=weight.data, transpose_a=True, mat_b=input, transpose_b=False, use_split_accumulator=False,
            out_dtype=out_dtype, bias=gemm_bias,
        )
        if len(ctx.in_shape) != 2:
            output = output.reshape(*ctx.in_shape[:-1], output.shape[-1])
        return output, phony

    @staticmethod
    @torch.no_grad()
    def backward(ctx, grad_output: torch.Tensor, grad_aux: torch.Tensor):
        input, weight, bias = ctx.saved_tensors
        module = ctx.module
        scaling = module.scaling if module is not None else None
        none = (None,) * 7
        if ctx.fp8_out:
            grad_output = grad_aux   # the gradient of the fp8 output arrives through its handle ...
            box = ctx.grad_box
            fp8_grad, arrivals = box.fp8_grad, box.arrivals
            box.fp8_grad, box.arrivals = None, 0
            if fp8_grad is not None:
                if arrivals > 1:
                    raise RuntimeError("an fp8 activation received gradients from more than one backward pass of its consumers, "
                                       "one of them in fp8: fp8 contributions cannot be summed.  Set `fp8_grad_input = False` "
                                       "on the consuming FP8Linear (high-precision gradients, summed by autograd), or give "
                                       "the producing layer a high-precision out_dtype")
                grad_output = fp8_grad   # ... or beside it, already quantised by the consumer's dgrad epilogue
        if grad_output is None:
            return none

        grad_bias = None
        if bias is not None and ctx.needs_input_grad[5]:
            # what autograd does for `output + bias` (linear.py:65): the gradient summed over the tokens (in fp32)
            g_hp = grad_output
            if type(g_hp) != torch.Tensor:
                from nanotron_amd.fp8.tensor import convert_tensor_from_fp8

                g_hp = convert_tensor_from_fp8(g_hp, g_hp.fp8_meta, bias.dtype)
            grad_bias = g_hp.reshape(-1, g_hp.shape[-1]).sum(0, dtype=torch.float32).to(bias.dtype)

        if type(grad_output) == torch.Tensor:
            g2d = grad_output.reshape(-1, grad_output.shape[-1]).contiguous()
            # wgrad reduces over the rows of dY: it needs the transposed bytes (kernel.py:44) unless the library reads
            # dY as it is, next to an input it also reads as it is
            x_plain = getattr(input, "_transposed", None) is None
            with_t = weight.requires_grad and not (
                x_plain and a_transposed_supported(g2d.shape[1], input.shape[1], g2d.shape[0]))
            grad_output = FP8Tensor(g2d, dtype=DTypes.FP8E5M2, state=scaling["output_grad"] if scaling else None,
                                    with_transpose=with_t)
        if module is not None and module.keep_quantised_grad:
            module.quantised_grad_output = grad_output   # for checkers: the e5m2 operand of dgrad and wgrad

        wants_dx = ctx.needs_input_grad[0] or (ctx.has_handle and ctx.needs_input_grad[6])
        grad_input = None
        box = ctx.input_box if wants_dx else None
        if box is not None:
            box.arrivals += 1
        fp8_dx = (box is not None and box.consumers == 1 and box.arrivals == 1 and box.state is not None
                  and box.state.known_initialised and module is not None and module.fp8_grad_input)
        # dX[M,K] = dY[M,N] . W[N,K]
        dgrad = dict(mat_a=weight.data, transpose_a=False, mat_b=grad_output, transpose_b=False, use_split_accumulator=True,
                     out_dtype=ctx.in_dtype or torch.float32)
        wgrad, slot = None, None
        if weight.requires_grad:
            # dW[N,K] = dY[M,N]^T . X[M,K].  The gradient is fp32 (kernel.py:24).  An fp32 parameter takes it as `.grad`
            # (side effect, as linear.py:110); a 16-bit parameter cannot hold an fp32 `.grad`, so there it is kept
            # beside the parameter as `.main_grad`, the fp32 master-gradient buffer an optimizer reads.
            slot = "grad" if weight.dtype == torch.float32 else "main_grad"
            acc = None
            if module is not None and module.accumulate_grad:
                prev = getattr(weight, slot, None)
                if prev is not None and prev.dtype == torch.float32:
                    acc = prev
            wgrad = dict(mat_a=input, transpose_a=False, mat_b=grad_output, transpose_b=True, use_split_accumulator=True,
                         accumulate_into=acc)
        grad_weight = None
        if fp8_dx:
            # dX leaves the dgrad epilogue as e5m2 bytes under the producer's output-gradient role (amax, history roll and
            # next scale included: what the producer's own quantisation of a high-precision dX would have done, minus
            # the rounding to the high-precision type in between); autograd carries a placeholder without memory
            box.fp8_grad = fp8_matmul_kernel(mat_a=weight.data, transpose_a=False, mat_b=grad_output, transpose_b=False,
                                             use_split_accumulator=True, out_dtype=DTypes.FP8E5M2, out_state=box.state)
            grad_input = torch.zeros(1, dtype=ctx.in_dtype or torch.float32, device=grad_output.device).expand(ctx.in_shape)
            module.fp8_grad_inputs_sent += 1
            if wgrad is not None:
                grad_weight = fp8_matmul_kernel(**wgrad)
        elif wants_dx and wgrad is not None:
            # the two GEMMs are independent: issued together they share kernel launches
            grad_input, grad_weight = fp8_matmul_pair(
                {k: v for k, v in dgrad.items() if k != "use_split_accumulator"},
                {k: v for k, v in wgrad.items() if k != "use_split_accumulator"})
        elif wants_dx:
            grad_input = fp8_matmul_kernel(**dgrad)
        elif wgrad is not None:
            grad_weight = fp8_matmul_kernel(**wgrad)
        if grad_input is not None and len(ctx.in_shape) != 2:
            grad_input = grad_input.reshape(ctx.in_shape)
        if grad_weight is not None:
            setattr(weight, slot, grad_weight)

        if ctx.has_handle:   # the input was an fp8 activation: its gradient goes to the handle that stands for it
            return None, None, None, None, None, grad_bias, grad_input
        return grad_input, None, None, None, None, grad_bias, None


def _frozen_copy(state: DelayedScaling) -> DelayedScaling:
    """A throw-away copy of a delayed-scaling state: the fp8-output GEMM of an evaluation pass casts with the held
    scale and does its bookkeeping on the copy."""
    c = DelayedScaling(state.dtype, state.history_len, state.margin, state._buf.device)
    c._buf.copy_(state._buf)
    c.initialised = state.initialised
    return c
