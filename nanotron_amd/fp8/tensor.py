"""FP8Tensor and the quantise / dequantise entry points (reference: src/nanotron/fp8/tensor.py).

The reference computes `amax` with two torch passes, the scale with ~8 scalar kernels and the cast
with Transformer Engine.  Here one C-ABI call does all of it on the device; amax, scale and the
delayed-scaling history never leave device memory.
"""
from __future__ import annotations

from typing import Optional, Union

import torch

from nanotron_amd import _native as nt
from nanotron_amd.fp8.constants import (
    DEFAULT_AMAX_HISTORY_LEN,
    DEFAULT_MARGIN,
    FP8_DTYPES,
    INITIAL_SCALING_FACTOR,
)
from nanotron_amd.fp8.dtypes import DType, DTypes

_FMT = {DTypes.FP8E4M3: nt.E4M3, DTypes.FP8E5M2: nt.E5M2}


def _int_margin(margin) -> int:
    m = float(margin)
    if not m.is_integer():
        raise ValueError(f"margin must be an integer number of binades, got {margin}")
    return int(m)


class DelayedScaling:
    """Per tensor-role delayed-scaling state kept on the device: `scale` (the scale the NEXT
    quantisation will use) and `amax_history` (newest first).  Not in the reference, whose
    FP8Tensor always scales from the current tensor (src/nanotron/fp8/tensor.py:25-28).

    The first quantisation through a fresh state (no finite positive amax recorded yet) uses
    current scaling, exactly the reference's behaviour; from then on every step is a single
    fused pass: cast with the held scale, amax, history roll, next scale.

    Whether a usable amax has been recorded is a flag in device memory, and the kernels of a role's first steps
    branch on it themselves: no quantisation reads anything back to the host.  The host learns of the flag
    through a copy that it does not wait for (`known_initialised`), and switches to the fused pass once it has;
    `initialised` is the exact answer and reads the flag if the host does not know yet."""

    def __init__(self, dtype: DTypes, history_len: int = DEFAULT_AMAX_HISTORY_LEN, margin: int = DEFAULT_MARGIN,
                 device: Union[str, torch.device] = "cuda"):
        assert isinstance(dtype, DTypes) and dtype in _FMT
        assert history_len >= 1
        self.dtype = dtype
        self.margin = _int_margin(margin)
        self.history_len = int(history_len)
        # one allocation: [scale, hist[0..H-1]]
        self._buf = torch.zeros(1 + self.history_len, dtype=torch.float32, device=device)
        self._buf[0] = INITIAL_SCALING_FACTOR
        self._flag = torch.zeros(1, dtype=torch.float32, device=device)   # 1.0 once a finite positive amax was recorded
        self._known = False      # the host has seen the flag set
        self._pending = None     # (pinned host copy of the flag, event behind the copy)

    @property
    def scale(self) -> torch.Tensor:
        return self._buf[0]

    @property
    def amax_history(self) -> torch.Tensor:
        return self._buf[1:]

    @property
    def known_initialised(self) -> bool:
        """True once the host has seen the device flag set; never waits.  False may be out of date by a few
        launches, which only means that the next quantisation still takes the two-launch first-use path."""
        if not self._known and self._pending is not None:
            host, event = self._pending
            if event.query():
                self._pending = None
                self._known = bool(host[0] != 0)
        return self._known

    def _watch_flag(self) -> None:
        """Queue a copy of the flag to pinned host memory behind the launches issued so far (not under graph capture,
        where a replay would write into memory the host polls at other times)."""
        if self._known or self._pending is not None or torch.cuda.is_current_stream_capturing():
            return
        host = torch.empty(1, dtype=torch.float32, pin_memory=True)
        host.copy_(self._flag, non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        self._pending = (host, event)

    @property
    def initialised(self) -> bool:
        if not self._known:
            self._pending = None
            self._known = bool(self._flag.item() != 0)
        return self._known

    @initialised.setter
    def initialised(self, value: bool) -> None:
        self._known = bool(value)
        self._pending = None
        self._flag.fill_(1.0 if value else 0.0)

    def state_dict(self):
        return {"buf": self._buf.clone(), "initialised": self.initialised}

    def load_state_dict(self, sd):
        self._buf.copy_(sd["buf"])
        self.initialised = bool(sd["initialised"])


class FP8Tensor(torch.Tensor):
    """uint8 tensor holding OCP fp8 bytes plus `fp8_meta` (reference: src/nanotron/fp8/tensor.py:9-36).

    `FP8Tensor(tensor, dtype)` is the reference call (current scaling).  Keyword-only extensions:
    `state` selects delayed scaling for a tensor role, `with_transpose` also produces the
    transposed bytes in the same pass (what the backward GEMMs consume), `update_state=False` quantises with the
    scale `state` holds but leaves the state as it is (evaluation passes between training steps)."""

    def __new__(cls, tensor: torch.Tensor, dtype: DTypes, *, state: Optional[DelayedScaling] = None,
                with_transpose: bool = False, margin: int = 0, update_state: bool = True) -> "FP8Tensor":
        assert isinstance(tensor, torch.Tensor), "tensor must be a tensor"
        assert tensor.dtype not in FP8_DTYPES, "The tensor already quantized to FP8"
        assert tensor.device != torch.device("cpu"), "FP8Tensor only supports CUDA device"
        assert isinstance(dtype, DTypes)
        if state is not None and not update_state:
            if state.initialised:
                return cast_with_scale(tensor, state.scale, dtype, with_transpose=with_transpose)
            return _quantize(cls, tensor, dtype, None, with_transpose, state.margin)
        return _quantize(cls, tensor, dtype, state, with_transpose, margin)

    def transposed(self) -> "FP8Tensor":
        """The [cols, rows] bytes as an FP8Tensor sharing this tensor's meta (reference:
        tex.fp8_transpose, src/nanotron/fp8/kernel.py:43-44).  Cached."""
        t = getattr(self, "_transposed", None)
        if t is None:
            assert self.dim() == 2, "transposed() needs a 2-D FP8Tensor"
            rows, cols = self.shape
            out = torch.empty((cols, rows), dtype=torch.uint8, device=self.device)
            src = self if self.is_contiguous() else self.contiguous()
            nt.check(nt.lib.ntfp8_transpose(src.data_ptr(), rows, cols, out.data_ptr(), nt.stream_ptr(self.device)),
                     "ntfp8_transpose")
            t = torch.Tensor._make_subclass(FP8Tensor, out)
            t.fp8_meta = self.fp8_meta
            self._transposed = t
        return t

    def __repr__(self) -> str:
        return f"FP8Tensor({self.as_subclass(torch.Tensor)}, fp8_meta={self.fp8_meta})"


def _quantize(cls, tensor: torch.Tensor, dtype: DTypes, state: Optional[DelayedScaling], with_transpose: bool,
              margin: int = 0) -> FP8Tensor:
    from nanotron_amd.fp8.meta import FP8Meta

    if dtype not in _FMT:
        raise ValueError(f"{dtype} is not an FP8 format")
    if tensor.dtype not in nt.TORCH_TO_NT:
        raise TypeError(f"cannot quantise a {tensor.dtype} tensor to FP8 (float32 / float16 / bfloat16 only)")
    if tensor.numel() == 0:
        raise RuntimeError("cannot quantise an empty tensor (amax of an empty tensor is undefined)")
    x = tensor.detach()
    if not x.is_contiguous():
        x = x.contiguous()
    dev = x.device
    if x.dim() >= 2:
        cols = x.shape[-1]
        rows = x.numel() // cols
    else:
        rows, cols = 1, x.numel()
    out = torch.empty(x.shape, dtype=torch.uint8, device=dev)
    out_t = None
    if with_transpose:
        assert x.dim() == 2, "with_transpose needs a 2-D tensor"
        out_t = torch.empty((cols, rows), dtype=torch.uint8, device=dev)
    scalars = torch.empty(2, dtype=torch.float32, device=dev)  # [amax, scale used]
    amax, scale = scalars[0], scalars[1]
    ws, st = nt.workspace_and_stream(dev)
    fmt = _FMT[dtype]
    xd = nt.TORCH_TO_NT[x.dtype]
    amax_p = scalars.data_ptr()
    scale_p = amax_p + 4
    if state is None:
        nt.check(nt.lib.ntfp8_quantize_current(x.data_ptr(), xd, rows, cols, fmt, _int_margin(margin), amax_p,
                                               scale_p, out.data_ptr(), nt.ptr(out_t), None, 0, None,
                                               ws.data_ptr(), st), "ntfp8_quantize_current")
    else:
        assert state.dtype == dtype, "delayed-scaling state was created for another format"
        assert state._buf.device == dev
        state_p = state._buf.data_ptr()   # [scale, hist[0..H-1]]
        if not state.known_initialised:
            # two launches that decide on the device: current scaling while the role holds no scale, the held scale once
            # it does (then with the results of the fused pass below, bit for bit)
            nt.check(nt.lib.ntfp8_quantize_first_use(x.data_ptr(), xd, rows, cols, fmt, state.margin, state_p, state_p + 4,
                                                     state.history_len, state._flag.data_ptr(), amax_p, scale_p,
                                                     out.data_ptr(), nt.ptr(out_t), ws.data_ptr(), st),
                     "ntfp8_quantize_first_use")
            state._watch_flag()
        else:
            nt.check(nt.lib.ntfp8_quantize_delayed(x.data_ptr(), xd, rows, cols, fmt, state.margin,
                                                   state_p, state_p + 4, state.history_len, amax_p, scale_p,
                                                   out.data_ptr(), nt.ptr(out_t), ws.data_ptr(), st),
                     "ntfp8_quantize_delayed")
    meta = FP8Meta(amax, scale, dtype)
    obj = torch.Tensor._make_subclass(cls, out)
    obj.fp8_meta = meta
    if out_t is not None:
        t = torch.Tensor._make_subclass(FP8Tensor, out_t)
        t.fp8_meta = meta
        obj._transposed = t
    return obj


@torch.no_grad()
def quantize_delayed_batch(tensors, dtype: DTypes, states, with_transpose) -> list:
    """[FP8Tensor(t, dtype, state=s, with_transpose=w) for t, s, w in zip(tensors, states, with_transpose)] for
    states that already hold a scale, through one library call (`ntfp8_quantize_delayed_batch`): tensors of one
    source type without a transposed copy share a launch, so that the end of one tensor's pass overlaps the
    beginning of the next.  Same results as the separate constructions, bit for bit."""
    from nanotron_amd.fp8.meta import FP8Meta

    tensors, states, with_transpose = list(tensors), list(states), list(with_transpose)
    assert len(tensors) == len(states) == len(with_transpose) and tensors
    dev = tensors[0].device
    fmt = _FMT[dtype]
    results = []
    for lo in range(0, len(tensors), 64):
        chunk = range(lo, min(lo + 64, len(tensors)))
        pool, st = nt.workspace_pool(dev, len(chunk))
        descs = (nt.QuantDesc * len(chunk))()
        keep = []
        for d, i in zip(descs, chunk):
            x, state = tensors[i].detach(), states[i]
            assert state.known_initialised and state.dtype == dtype and state._buf.device == dev and x.device == dev
            assert x.dtype in nt.TORCH_TO_NT and x.numel() > 0
            if not x.is_contiguous():
                x = x.contiguous()
            cols = x.shape[-1] if x.dim() >= 2 else x.numel()
            rows = x.numel() // cols
            out = torch.empty(x.shape, dtype=torch.uint8, device=dev)
            out_t = None
            if with_transpose[i]:
                assert x.dim() == 2, "with_transpose needs a 2-D tensor"
                out_t = torch.empty((cols, rows), dtype=torch.uint8, device=dev)
            scalars = torch.empty(2, dtype=torch.float32, device=dev)  # [amax, scale used]
            state_p = state._buf.data_ptr()
            d.x, d.x_dtype, d.fmt, d.margin, d.history_len = x.data_ptr(), nt.TORCH_TO_NT[x.dtype], fmt, state.margin, state.history_len
            d.rows, d.cols = rows, cols
            d.scale_state, d.amax_history = state_p, state_p + 4
            d.amax_out, d.scale_used_out = scalars.data_ptr(), scalars.data_ptr() + 4
            d.out, d.out_t, d.workspace = out.data_ptr(), nt.ptr(out_t), pool[i - lo].data_ptr()
            keep.append((x, out, out_t, scalars))
        nt.check(nt.lib.ntfp8_quantize_delayed_batch(descs, len(chunk), st), "ntfp8_quantize_delayed_batch")
        for x, out, out_t, scalars in keep:
            meta = FP8Meta(scalars[0], scalars[1], dtype)
            obj = torch.Tensor._make_subclass(FP8Tensor, out)
            obj.fp8_meta = meta
            if out_t is not None:
                t = torch.Tensor._make_subclass(FP8Tensor, out_t)
                t.fp8_meta = meta
                obj._transposed = t
            results.append(obj)
    return results


def cast_with_scale(tensor: torch.Tensor, scale: torch.Tensor, dtype: DTypes, with_transpose: bool = False) -> FP8Tensor:
    """FP8Tensor of `tensor` cast with a given device scale (no amax pass, no delayed-scaling state touched):
    the cast half of the reference's FP8Tensor.__new__ (src/nanotron/fp8/tensor.py:28,60-65).  Used to
    rebuild an fp8 copy exactly as it was, e.g. after loading a checkpoint."""
    from nanotron_amd.fp8.meta import FP8Meta

    x = tensor.detach()
    if not x.is_contiguous():
        x = x.contiguous()
    dev = x.device
    assert dev != torch.device("cpu"), "cast_with_scale only supports CUDA tensors"
    cols = x.shape[-1] if x.dim() >= 2 else x.numel()
    rows = x.numel() // cols
    scalars = torch.zeros(2, dtype=torch.float32, device=dev)  # [amax (not computed), scale]
    scalars[1].copy_(scale.reshape(()).to(device=dev, dtype=torch.float32))
    out = torch.empty(x.shape, dtype=torch.uint8, device=dev)
    out_t = None
    if with_transpose:
        assert x.dim() == 2, "with_transpose needs a 2-D tensor"
        out_t = torch.empty((cols, rows), dtype=torch.uint8, device=dev)
    nt.check(nt.lib.ntfp8_cast_to_fp8(x.data_ptr(), nt.TORCH_TO_NT[x.dtype], rows, cols, scalars[1].data_ptr(), _FMT[dtype],
                                      out.data_ptr(), nt.ptr(out_t), nt.stream_ptr(dev)), "ntfp8_cast_to_fp8")
    meta = FP8Meta(scalars[0], scalars[1], dtype)
    obj = torch.Tensor._make_subclass(FP8Tensor, out)
    obj.fp8_meta = meta
    if out_t is not None:
        t = torch.Tensor._make_subclass(FP8Tensor, out_t)
        t.fp8_meta = meta
        obj._transposed = t
    return obj


def convert_torch_dtype_to_te_dtype(dtype) -> DType:
    """Reference: src/nanotron/fp8/tensor.py:39-55 (same key set, returns this library's enum)."""
    mapping = {
        torch.int32: "kInt32",
        torch.float32: "kFloat32",
        torch.float16: "kFloat16",
        torch.bfloat16: "kBFloat16",
        DTypes.FP8E4M3: "kFloat8E4M3",
        DTypes.FP8E5M2: "kFloat8E5M2",
        DTypes.KFLOAT16: "kFloat16",
    }
    return getattr(DType, mapping[dtype])


def convert_tensor_to_fp8(tensor: torch.Tensor, meta) -> torch.Tensor:
    """Cast with the scale held in `meta` (reference: src/nanotron/fp8/tensor.py:60-65,
    tex.cast_to_fp8).  Returns the uint8 bytes.  meta.amax is left untouched: at the reference's
    only call site it already equals max|x| (tensor.py:25-28), so TE's amax update is a no-op."""
    assert tensor.device != torch.device("cpu"), "convert_tensor_to_fp8 only supports CUDA tensors"
    x = tensor.detach().contiguous()
    dev = x.device
    scale = meta.scale
    if not (isinstance(scale, torch.Tensor) and scale.device == dev and scale.dtype == torch.float32):
        scale = torch.as_tensor(scale, dtype=torch.float32).to(dev)
    scale = scale.reshape(())
    cols = x.shape[-1] if x.dim() >= 2 else x.numel()
    rows = x.numel() // cols
    out = torch.empty(x.shape, dtype=torch.uint8, device=dev)
    nt.check(nt.lib.ntfp8_cast_to_fp8(x.data_ptr(), nt.TORCH_TO_NT[x.dtype], rows, cols, scale.data_ptr(),
                                      _FMT[meta.dtype], out.data_ptr(), None, nt.stream_ptr(dev)), "ntfp8_cast_to_fp8")
    return out


def convert_tensor_from_fp8(tensor: torch.Tensor, meta, dtype: torch.dtype) -> torch.Tensor:
    """Dequantise (reference: src/nanotron/fp8/tensor.py:68-74, tex.cast_from_fp8)."""
    assert isinstance(tensor, torch.Tensor)
    assert isinstance(dtype, torch.dtype)
    assert tensor.device != torch.device("cpu"), "convert_tensor_from_fp8 only supports CUDA tensors"
    if dtype not in nt.TORCH_TO_NT:
        raise TypeError(f"unsupported output dtype {dtype}")
    q = tensor.as_subclass(torch.Tensor) if isinstance(tensor, FP8Tensor) else tensor
    q = q.contiguous()
    dev = q.device
    scale = meta.scale
    if not (isinstance(scale, torch.Tensor) and scale.device == dev and scale.dtype == torch.float32):
        scale = torch.as_tensor(scale, dtype=torch.float32).to(dev)
    out = torch.empty(q.shape, dtype=dtype, device=dev)
    if q.numel():
        nt.check(nt.lib.ntfp8_cast_from_fp8(q.data_ptr(), _FMT[meta.dtype], scale.data_ptr(), q.numel(), out.data_ptr(),
                                            nt.TORCH_TO_NT[dtype], nt.stream_ptr(dev)), "ntfp8_cast_from_fp8")
    return out


def update_scaling_factor(amax: torch.Tensor, scaling_factor: torch.Tensor, dtype: DTypes,
                          margin: float = 0) -> torch.Tensor:
    """Power-of-two scale from an amax (reference: src/nanotron/fp8/tensor.py:77-105).

    Device tensors are processed by the HIP kernel and the result stays on the device; when both
    arguments are host tensors (as in FP8Linear.__init__, src/nanotron/fp8/linear.py:33-42) the
    native library evaluates the same function on the host."""
    assert amax.dtype == torch.float32
    assert scaling_factor.dtype == torch.float32
    fmt = _FMT[dtype]
    m = _int_margin(margin)
    if not amax.is_cuda and not scaling_factor.is_cuda:
        a, s = torch.broadcast_tensors(amax, scaling_factor)
        flat = [nt.update_scaling_factor_host(float(x), float(y), fmt, m)
                for x, y in zip(a.reshape(-1).tolist(), s.reshape(-1).tolist())]
        return torch.tensor(flat, dtype=torch.float32).reshape(a.shape)
    dev = amax.device if amax.is_cuda else scaling_factor.device
    a, s = torch.broadcast_tensors(amax.to(dev), scaling_factor.to(dev))
    a, s = a.contiguous(), s.contiguous()
    out = torch.empty_like(a)
    if a.numel():
        nt.check(nt.lib.ntfp8_update_scaling_factor(a.data_ptr(), s.data_ptr(), fmt, m, out.data_ptr(), a.numel(),
                                                    nt.stream_ptr(dev)), "ntfp8_update_scaling_factor")
    return out
