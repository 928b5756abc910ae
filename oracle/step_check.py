"""Checker for the benchmark's headline workload.  TEST INFRASTRUCTURE ONLY (used by tests/ and by
bench.py's correctness gate; the product never imports it).

Workload (benchmark configuration 5): the Llama-3-8B decoder-block linears at 4096 tokens, forward + backward with
per-tensor delayed scaling (amax history 16, margin 0) over several steps; fresh seeded activations and output
gradients every step, the master weights perturbed every step so that the weight role's amax history moves.

What is compared after every layer of every step, product path (FP8Linear on the GPU) against the CPU oracle:
  * bit-exact: the scale used, the amax, the next scale and the whole amax history of the three tensor roles
    (input e4m3, weight e4m3, output gradient e5m2); the fp8 bytes of the weight, of the quantised input and of the
    quantised output gradient;
  * Y and dX (bf16 outputs) on sampled rows against the oracle's fp32 result rounded once to bf16, and dW (fp32,
    optionally added to a pre-filled fp32 master-gradient buffer) on sampled rows against the oracle: rel-L2 <= 1e-3.
The GEMM semantics follow src/nanotron/fp8/linear.py:69-112 (forward X.W^T; backward dY.W and dY^T.X) and
src/nanotron/fp8/kernel.py:46-68 (fp32 accumulation, one descale).
"""
from __future__ import annotations

from typing import Dict, List

import torch

from oracle import fp8_oracle as O

TOKENS = 4096
LINEARS = [  # name, in_features (K), out_features (N)
    ("qkv", 4096, 6144),
    ("o", 4096, 4096),
    ("gate", 4096, 14336),
    ("up", 4096, 14336),
    ("down", 14336, 4096),
]
SEED = 1234 + 500
REL_L2_F32 = 1e-3    # stated GEMM tolerance against fp32 matmul of exactly-upcast operands
REL_L2_BF16 = 1e-3   # bf16 outputs against the oracle's result rounded once to bf16
ROLES = ("input", "weight", "output_grad")


def initial_weight(i: int, K: int, N: int) -> torch.Tensor:
    return O.normal_tensor(SEED + 10 + i, (N, K), 0.02, torch.bfloat16)


def perturbed_weight(w: torch.Tensor, step: int, i: int) -> torch.Tensor:
    """The master weight of layer i after `step`'s stand-in for an optimizer update."""
    d = O.normal_tensor(SEED + 9000 + 16 * step + i, tuple(w.shape), 0.002 * (1 + step % 3), torch.float32)
    return (w.float() + d).to(torch.bfloat16)


def step_inputs(step: int, i: int, K: int, N: int, tokens: int = TOKENS):
    """(X bf16 [tokens, K], dY bf16 [tokens, N]) of layer i at `step`; the spread changes with the step so that
    the amax histories of the activation roles move as well."""
    x = O.normal_tensor(SEED + 1000 + 16 * step + i, (tokens, K), 1.0 + 0.25 * (step % 4), torch.bfloat16)
    gy = O.normal_tensor(SEED + 5000 + 16 * step + i, (tokens, N), 1e-3 * (1 + step % 2), torch.bfloat16)
    return x, gy


def new_reference_state() -> List[Dict[str, O.DelayedScaling]]:
    return [{"input": O.DelayedScaling(O.E4M3), "weight": O.DelayedScaling(O.E4M3), "output_grad": O.DelayedScaling(O.E5M2)}
            for _ in LINEARS]


def _rows(n: int, step: int, i: int) -> torch.Tensor:
    g = torch.Generator().manual_seed(77 + 16 * step + i)
    fixed = [0, 1, 127, 128, 255, 256, n // 2 - 1, n // 2, n - 257, n - 256, n - 129, n - 1]
    rnd = torch.randint(0, n, (6,), generator=g).tolist()
    return torch.tensor(sorted({r for r in fixed + rnd if 0 <= r < n}))


def _bits(t: torch.Tensor) -> torch.Tensor:
    return t.detach().float().cpu().contiguous().view(torch.int32)


def check_layer(tag: str, lin, ref: Dict[str, O.DelayedScaling], x: torch.Tensor, w: torch.Tensor, gy: torch.Tensor,
                y_gpu: torch.Tensor, dx_gpu: torch.Tensor, dw_gpu: torch.Tensor, xq_gpu, step: int, i: int,
                dw_base: torch.Tensor = None, gq_gpu=None) -> dict:
    """Advances the oracle's three roles of this layer by one step and compares; raises AssertionError naming what
    differs.  `xq_gpu` is the FP8Tensor of the input that the layer saved for its backward; `dw_base` (CPU, fp32) is
    what the weight-gradient buffer held before this backward when the layer accumulates into it
    (src/nanotron/optim/gradient_accumulator.py:222); `gq_gpu` is the FP8Tensor of the output gradient that the backward
    GEMMs read (src/nanotron/fp8/linear.py:99-102), compared like the input when given."""
    xq, wq, gq = ref["input"].quantise(x), ref["weight"].quantise(w), ref["output_grad"].quantise(gy)
    for role, q in (("input", xq), ("weight", wq), ("output_grad", gq)):
        st, rf = lin.scaling[role], ref[role]
        assert torch.equal(_bits(st.scale), _bits(rf.scale)), f"{tag} {role}: next scale {st.scale.item()} != {rf.scale.item()}"
        assert torch.equal(_bits(st.amax_history), _bits(rf.hist)), f"{tag} {role}: amax history differs"
    wg = lin.weight.data
    operands = [("weight", wg, wq), ("input", xq_gpu, xq)]
    if gq_gpu is not None:
        operands.append(("output gradient", gq_gpu, gq))
    for name, got, q in operands:
        assert torch.equal(_bits(got.fp8_meta.amax), _bits(q.amax)), f"{tag} {name}: amax {got.fp8_meta.amax.item()} != {q.amax.item()}"
        assert torch.equal(_bits(got.fp8_meta.scale), _bits(q.scale)), f"{tag} {name}: scale used {got.fp8_meta.scale.item()} != {q.scale.item()}"
        same = torch.equal(got.as_subclass(torch.Tensor), q.q.to(got.device))
        assert same, f"{tag} {name}: fp8 bytes differ from the oracle"
    M, K = x.shape
    N = w.shape[0]
    xf, wf, gf = O.upcast(xq.q, O.E4M3), O.upcast(wq.q, O.E4M3), O.upcast(gq.q, O.E5M2)
    ax = (1 / xq.scale) * (1 / wq.scale)
    ag = (1 / gq.scale) * (1 / wq.scale)
    aw = (1 / gq.scale) * (1 / xq.scale)
    rm = _rows(M, step, i)
    y_ref = (xf[rm] @ wf.t()) * ax                    # linear.py:82-84
    dx_ref = (gf[rm] @ wf) * ag                       # linear.py:104-106 as documented at linear.py:92-96
    rn = _rows(N, step, i)
    dw_ref = (gf[:, rn].t().contiguous() @ xf) * aw   # linear.py:107-109
    dw_got = dw_gpu[rn.to(dw_gpu.device)].float().cpu()
    if dw_base is not None:
        # the buffer's old content is much larger than the gradient: take it off again (the fp32 add costs 2^-24 of
        # the buffer's value, far below the tolerance) so that the tolerance applies to the gradient itself
        dw_got = dw_got - dw_base[rn]
    e_y = O.rel_l2(y_gpu[rm.to(y_gpu.device)].float().cpu(), y_ref.to(torch.bfloat16).float())
    e_dx = O.rel_l2(dx_gpu[rm.to(dx_gpu.device)].float().cpu(), dx_ref.to(torch.bfloat16).float())
    e_dw = O.rel_l2(dw_got, dw_ref)
    assert y_gpu.dtype == torch.bfloat16 and dx_gpu.dtype == torch.bfloat16 and dw_gpu.dtype == torch.float32
    assert e_y <= REL_L2_BF16, f"{tag} forward: rel-L2 {e_y:.3e} > {REL_L2_BF16}"
    assert e_dx <= REL_L2_BF16, f"{tag} dgrad: rel-L2 {e_dx:.3e} > {REL_L2_BF16}"
    assert e_dw <= REL_L2_F32, f"{tag} wgrad: rel-L2 {e_dw:.3e} > {REL_L2_F32}"
    return {"fwd": e_y, "dgrad": e_dx, "wgrad": e_dw}
