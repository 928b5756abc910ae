"""A seeded random sweep of FP8Tensor quantisation through the product path (src/nanotron/fp8/tensor.py:12-33 with the
delayed-scaling extension): 1-D / 2-D / 3-D shapes of any size, three source types, both formats, current and delayed
scaling over several steps, transposed copies, views that start 2 - 12 bytes off an aligned address, all-zero first
steps, NaN / Inf entries, tiny and huge magnitudes.  Bytes, transposed bytes, amax, scale, next scale and history are
compared with the CPU oracle bit for bit."""
import random

import pytest
import torch

from oracle import fp8_oracle as O

pytestmark = pytest.mark.gpu


def same(a, b):
    a, b = a.detach().float().cpu().reshape(-1), b.detach().float().cpu().reshape(-1)
    return bool(torch.all((a.view(torch.int32) == b.view(torch.int32)) | (a.isnan() & b.isnan())))


@pytest.mark.parametrize("seed", [21, 22])
def test_random_quantisations_against_the_oracle(seed):
    from nanotron_amd.fp8 import DelayedScaling, DTypes, FP8Tensor

    dev = torch.device("cuda", 0)
    rng = random.Random(seed)
    bad = []
    for case in range(60):
        nd = rng.choice([1, 2, 2, 2, 3])
        if nd == 1: shape = (rng.randrange(1, 70000),)
        elif nd == 2: shape = (rng.randrange(1, 1500), rng.randrange(1, 1500))
        else: shape = (rng.randrange(1, 9), rng.randrange(1, 300), rng.randrange(1, 300))
        dt = rng.choice([torch.bfloat16, torch.float16, torch.float32])
        fmt = rng.choice([O.E4M3, O.E5M2])
        delayed = rng.random() < 0.6
        steps = rng.randrange(1, 6) if delayed else 1
        wt = nd == 2 and rng.random() < 0.5
        special = rng.choice(["none", "none", "zero", "nan", "inf", "tiny", "huge"])
        offset = rng.choice([0, 0, 1, 3])   # misaligned view
        print(f"seed {seed} case {case}: shape={shape} dt={dt} fmt={fmt} delayed={delayed} steps={steps} wt={wt} special={special} off={offset}", flush=True)
        st = DelayedScaling(DTypes.FP8E4M3 if fmt == O.E4M3 else DTypes.FP8E5M2, 16, 0, dev) if delayed else None
        ref = O.DelayedScaling(fmt) if delayed else None
        for step in range(steps):
            g = torch.Generator().manual_seed((seed * 1000 + case) * 100 + step)
            n = 1
            for s_ in shape: n *= s_
            base = torch.randn(n + offset, generator=g) * (10.0 ** rng.uniform(-3, 3))
            if special == "zero" and step == 0: base.zero_()
            if special == "tiny": base *= 1e-30
            if special == "huge": base *= 1e30
            base = base.to(dt)
            if special == "nan" and step == steps - 1: base[offset + rng.randrange(n)] = float("nan")
            if special == "inf" and step == steps - 1: base[offset + rng.randrange(n)] = float("inf")
            x_cpu = base[offset:].reshape(shape)
            x = base.to(dev)[offset:].reshape(shape)
            q = FP8Tensor(x, DTypes.FP8E4M3 if fmt == O.E4M3 else DTypes.FP8E5M2, state=st, with_transpose=wt)
            r = ref.quantise(x_cpu) if delayed else O.quantise_current(x_cpu, fmt)
            ok = torch.equal(q.as_subclass(torch.Tensor).cpu(), r.q) and same(q.fp8_meta.amax, r.amax) and same(q.fp8_meta.scale, r.scale)
            if wt: ok = ok and torch.equal(q._transposed.as_subclass(torch.Tensor).cpu(), r.q.t().contiguous())
            if delayed:
                ok = ok and same(st._buf[0], ref.scale) and same(st._buf[1:], ref.hist) and st.initialised == ref.initialised
            if not ok:
                bad.append((case, step, shape, str(dt), fmt, delayed, wt, special, offset))
                break
    assert not bad, bad
