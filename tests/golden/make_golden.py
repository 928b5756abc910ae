"""Writes tests/golden/fp8_golden.npz: known answers for the FP8 path, derived with exact rational
arithmetic from the definitions alone (OCP FP8 formats; the scale formula of
src/nanotron/fp8/tensor.py:97-103; the delayed-scaling rules the benchmark configurations fix).

Nothing here imports the oracle, the package under test, torch or the reference: the file is an
independent third statement of the arithmetic, so that a mistake shared by the oracle and the kernels
(a wrong bias, a tie rounded the wrong way, an off-by-one in the history roll) still fails a test.
The reference ships no golden vectors for this path (its tests draw unseeded random inputs), which is
why these are computed rather than copied.

    python tests/golden/make_golden.py        # rewrites fp8_golden.npz next to this file
"""
import math
import os
import random
import struct
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
FP8_MAX = {0: Fraction(448), 1: Fraction(57344)}  # 0 = e4m3fn, 1 = e5m2


# ------------------------------------------------------------------ OCP FP8 decode, by the definition
def decode(fmt: int, byte: int):
    """Value of an fp8 code as a Fraction, or 'nan' / 'inf' / '-inf'."""
    s = -1 if byte & 0x80 else 1
    if fmt == 0:  # e4m3fn: bias 7, no infinities, S.1111.111 is NaN
        e, m = (byte >> 3) & 0xF, byte & 0x7
        if e == 15 and m == 7:
            return "nan"
        mag = Fraction(m, 8) * Fraction(2) ** -6 if e == 0 else (1 + Fraction(m, 8)) * Fraction(2) ** (e - 7)
    else:  # e5m2: bias 15, IEEE-like specials
        e, m = (byte >> 2) & 0x1F, byte & 0x3
        if e == 31:
            return "nan" if m else ("inf" if s > 0 else "-inf")
        mag = Fraction(m, 4) * Fraction(2) ** -14 if e == 0 else (1 + Fraction(m, 4)) * Fraction(2) ** (e - 15)
    return s * mag


def decode_f32(fmt: int, byte: int) -> np.float32:
    v = decode(fmt, byte)
    if v == "nan":
        return np.float32(np.nan)
    if v == "inf":
        return np.float32(np.inf)
    if v == "-inf":
        return np.float32(-np.inf)
    f = np.float32(float(v))
    if byte & 0x80 and v == 0:
        f = np.float32(-0.0)
    return f


FINITE = {f: sorted((decode(f, b), b) for b in range(0x80) if not isinstance(decode(f, b), str)) for f in (0, 1)}


# ------------------------------------------------------------------ saturating round-to-nearest-even encode
def encode(fmt: int, x: float, scale: float) -> int:
    """Byte for fp32 x times a power-of-two fp32 scale (so the fp32 product is exact unless it leaves the
    fp32 range, which the chosen inputs avoid): clamp to +-fp8_max, nearest code, ties to the even code."""
    if math.isnan(x):
        return 0xFF if math.copysign(1.0, x) < 0 else 0x7F
    neg = math.copysign(1.0, x) < 0
    if math.isinf(x):
        mag = FP8_MAX[fmt]
    else:
        mag = min(abs(Fraction(x) * Fraction(scale)), FP8_MAX[fmt])
    best = None
    for v, b in FINITE[fmt]:
        d = abs(v - mag)
        if best is None or d < best[0] or (d == best[0] and b % 2 == 0 and best[1] % 2 == 1):
            best = (d, b)
    return best[1] | (0x80 if neg else 0)


# ------------------------------------------------------------------ scale (src/nanotron/fp8/tensor.py:97-103)
F32_MAX = Fraction(2) ** 128 - Fraction(2) ** 104
F32_OVER = Fraction(2) ** 128 - Fraction(2) ** 103  # quotients at or above this round to +Inf in fp32


def scale_exponent(fmt: int, amax: Fraction):
    """k with scale = 2^k for a finite positive amax whose quotient is far from a power of two (true for
    every 16-bit amax: 8 or 11 significant bits), or None when the fp32 quotient overflows (scale = +Inf)."""
    q = FP8_MAX[fmt] / amax
    if q >= F32_OVER:
        return None
    k = 0
    while Fraction(2) ** (k + 1) <= q:
        k += 1
    while Fraction(2) ** k > q:
        k -= 1
    return k


def bf16_to_float(bits: int) -> float:
    return struct.unpack("<f", struct.pack("<I", bits << 16))[0]


def f32(x) -> np.float32:
    return np.float32(x)


def scale_value(fmt: int, amax: float, old: float) -> np.float32:
    """The literal formula on special inputs, the closed form otherwise."""
    if math.isnan(amax) or amax <= 0.0:
        return f32(old)
    if math.isinf(amax):
        return f32(1.0) / f32(old)  # log2(0) = -inf: the "exp < 0" branch inverts the held scale
    k = scale_exponent(fmt, Fraction(amax))
    return f32(np.inf) if k is None else f32(2.0) ** f32(k)


# ------------------------------------------------------------------ delayed scaling (history newest first)
def delayed_sequence(fmt: int, amaxes, hist_len: int):
    hist = [0.0] * hist_len
    scale = 1.0
    seen = False
    used, nxt, hists = [], [], []
    for a in amaxes:
        s_t = float(scale_value(fmt, a, 1.0)) if not seen else scale
        if not seen and (a > 0.0 and not math.isinf(a) and not math.isnan(a)):
            seen = True
        hist = [a] + hist[:-1]
        m = float("nan") if any(math.isnan(h) for h in hist) else max(hist)
        scale = float(scale_value(fmt, m, s_t))
        used.append(s_t)
        nxt.append(scale)
        hists.append(list(hist))
    return used, nxt, hists


def main():
    out = {}
    for fmt, name in ((0, "e4m3"), (1, "e5m2")):
        out[f"decode_{name}"] = np.array([decode_f32(fmt, b) for b in range(256)], dtype=np.float32)

    # every positive finite bf16 amax: exponent of the scale (32767 marks +Inf)
    bits = np.array([b for b in range(1, 0x7F80)], dtype=np.uint16)
    out["scale_amax_bf16_bits"] = bits
    for fmt, name in ((0, "e4m3"), (1, "e5m2")):
        ks = []
        for b in bits:
            k = scale_exponent(fmt, Fraction(bf16_to_float(int(b))))
            ks.append(32767 if k is None else k)
        out[f"scale_exp_{name}"] = np.array(ks, dtype=np.int16)
    # special amax values: [amax, old scale] -> scale, both formats
    specials = [(0.0, 1.0), (0.0, 8.0), (-1.0, 4.0), (float("nan"), 2.0), (float("inf"), 1.0), (float("inf"), 4.0),
                (1.0, 1.0), (448.0, 1.0), (57344.0, 1.0), (3.3895313892515355e38, 1.0), (1e-38, 1.0)]
    out["scale_special_in"] = np.array(specials, dtype=np.float32)
    for fmt, name in ((0, "e4m3"), (1, "e5m2")):
        out[f"scale_special_{name}"] = np.array([scale_value(fmt, float(np.float32(a)), o) for a, o in specials],
                                                dtype=np.float32)

    # casts: specials, every tie between neighbouring codes, the codes themselves, seeded random values
    rng = random.Random(20240607)
    for fmt, name in ((0, "e4m3"), (1, "e5m2")):
        xs, ss = [], []
        for x in (float("nan"), -float("nan"), float("inf"), -float("inf"), 0.0, -0.0, 1e-30, -1e-30, 17.0, 19.0, 21.0,
                  23.0, 464.0, 465.0, 1e9, -1e9):
            for s in (1.0, 0.125, 32.0):
                xs.append(x)
                ss.append(s)
        vals = [v for v, _ in FINITE[fmt]]
        for lo, hi in zip(vals[:-1], vals[1:]):
            mid = (lo + hi) / 2
            for v in (lo, mid, hi):
                for sgn in (1, -1):
                    xs.append(sgn * float(v))  # exact in fp32: at most 5 significant bits
                    ss.append(1.0)
                    xs.append(sgn * float(v) * 8.0)
                    ss.append(0.125)
        for _ in range(3000):
            e = rng.uniform(-20, 18)
            x = struct.unpack("<f", struct.pack("<f", rng.choice((-1, 1)) * 2.0 ** e * rng.uniform(1, 2)))[0]
            xs.append(x)
            ss.append(rng.choice((1.0, 0.125, 32.0, 2.0 ** -10)))
        out[f"cast_x_{name}"] = np.array(xs, dtype=np.float32)
        out[f"cast_scale_{name}"] = np.array(ss, dtype=np.float32)
        out[f"cast_bytes_{name}"] = np.array([encode(fmt, float(np.float32(x)), s) for x, s in zip(xs, ss)], dtype=np.uint8)

    # delayed scaling over 12 steps, history 4: growth, decay past the history, zero tensor, NaN tensor
    amaxes = [3.0, 0.5, 100.0, 0.25, 0.25, 0.25, 0.25, 0.0, float("nan"), 7.0, 7.0, 2000.0, 1.0, 1.0, 1.0, 1.0]
    out["delayed_amax"] = np.array(amaxes, dtype=np.float32)
    for fmt, name in ((0, "e4m3"), (1, "e5m2")):
        used, nxt, hists = delayed_sequence(fmt, amaxes, 4)
        out[f"delayed_used_{name}"] = np.array(used, dtype=np.float32)
        out[f"delayed_next_{name}"] = np.array(nxt, dtype=np.float32)
        out[f"delayed_hist_{name}"] = np.array(hists, dtype=np.float32)

    # integer GEMM: operands exactly representable in both formats, exact integer result
    a = np.array([[rng.choice((-4, -3, -2, -1, 0, 1, 2, 3, 4)) for _ in range(160)] for _ in range(48)], dtype=np.int32)
    b = np.array([[rng.choice((-4, -3, -2, -1, 0, 1, 2, 3, 4)) for _ in range(160)] for _ in range(40)], dtype=np.int32)
    out["gemm_a"] = a.astype(np.float32)
    out["gemm_b"] = b.astype(np.float32)
    out["gemm_d"] = (a @ b.T).astype(np.float32)

    np.savez_compressed(os.path.join(HERE, "fp8_golden.npz"), **out)
    print("wrote", os.path.join(HERE, "fp8_golden.npz"), {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
