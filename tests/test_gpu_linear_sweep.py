"""A seeded random sweep of FP8Linear forward + backward over three delayed-scaling steps each (the product path of
src/nanotron/fp8/linear.py:51-112): token counts and feature sizes that are multiples of 256, of 16, or of nothing, with
and without accumulation into the fp32 master gradient.  Whatever route the host picks (operands read untransposed,
transposed copies, the 128-tile or the one-output-per-thread kernel), scaling state and fp8 bytes must equal the
oracle's bit for bit and Y, dX, dW must be within rel-L2 1e-3 (oracle/step_check.py holds the comparison the full-size
configuration test uses)."""
import random

import pytest
import torch

from oracle import step_check as C

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [31, 32])
def test_random_linears_against_the_oracle(seed):
    from nanotron_amd.fp8 import DTypes, FP8Linear, FP8Parameter
    from nanotron_amd.fp8.optim import requantize_fp8_weights

    rng = random.Random(seed)
    bad = []
    for case in range(16):
        kind = rng.choice(["aligned", "aligned", "mult16", "odd"])
        if kind == "aligned": T, K, N = rng.choice([256, 512, 1024, 2048]), rng.choice([256, 512, 1024, 1536]), rng.choice([256, 768, 1024, 2304])
        elif kind == "mult16": T, K, N = 16 * rng.randrange(9, 80), 16 * rng.randrange(16, 70), 16 * rng.randrange(9, 90)
        else: T, K, N = rng.randrange(1, 700), rng.randrange(1, 600), rng.randrange(1, 600)
        acc = rng.random() < 0.4
        print(f"seed {seed} case {case}: {kind} T={T} K={K} N={N} acc={acc}", flush=True)
        lin = FP8Linear(K, N, bias=False, device="cuda", out_dtype=torch.bfloat16, delayed_scaling=True, amax_history_len=16, margin=0, accumulate_grad=acc)
        w = C.initial_weight(case, K, N)
        lin.weight = FP8Parameter(w.cuda(), DTypes.FP8E4M3)
        ref = C.new_reference_state()[0]
        try:
            for step in range(3):
                w = C.perturbed_weight(w, step, case)
                with torch.no_grad():
                    lin.weight.as_subclass(torch.Tensor).copy_(w.cuda())
                requantize_fp8_weights([lin])
                x, gy = C.step_inputs(step, case, K, N, tokens=T)
                xg = x.cuda().requires_grad_(True)
                base = lin.weight.main_grad.clone().cpu() if (acc and getattr(lin.weight, "main_grad", None) is not None) else None
                y = lin(xg)
                xq_gpu = y.grad_fn.saved_tensors[0]
                y.backward(gy.cuda())
                C.check_layer(f"case {case} step {step}", lin, ref, x, w, gy, y.detach(), xg.grad, lin.weight.main_grad, xq_gpu, step, case, dw_base=base)
        except AssertionError as e:
            bad.append((case, kind, T, K, N, acc, str(e)[:200]))
    assert not bad, bad
