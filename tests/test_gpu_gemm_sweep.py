"""A seeded random sweep of `ntfp8_gemm_batch` requests through the C ABI: every kernel path (256-tile, half-tile tail,
128-tile, one-output-per-thread), both operand formats on either side, operands given plain or as their transposes,
all output types including fp8 with its transposed copy and amax, fp32 accumulation, bias, scales given as scales or
as inverse scales, ragged and tiny shapes.  Reference: an fp64 product of the exactly-upcast operands (the oracle's
decode table), rel-L2 <= 1e-3 as the GEMM gate everywhere in this suite (4e-3 for bf16 outputs, whose own rounding
is 2^-9 relative), bit equality for integer-valued operands with fp32 outputs, and for fp8 outputs bit equality with
the stand-alone cast of the same kernel's fp32 result.  (src/nanotron/fp8/kernel.py:46-68 is the call it serves.)"""
import random

import pytest
import torch

from oracle import fp8_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_requests_against_fp64_reference(seed):
    from nanotron_amd import _native as nt

    dev = torch.device("cuda", 0)
    rng = random.Random(seed)
    tabs = {f: torch.tensor(O.decode_table(f), dtype=torch.float64, device=dev) for f in (O.E4M3, O.E5M2)}
    st = nt.stream_ptr(dev)
    ws, _ = nt.workspace_and_stream(dev)
    TD = {nt.F32: torch.float32, nt.F16: torch.float16, nt.BF16: torch.bfloat16}
    bad = []
    for case in range(60):
        kind = rng.choice(["big", "big", "edge", "small", "odd"])
        if kind == "big":
            M, N, K = rng.choice([256, 272, 512, 768, 1040, 1280]), rng.choice([256, 288, 512, 784, 1024, 1536]), rng.choice([256, 384, 512, 1024, 2064])
        elif kind == "edge":
            M, N, K = rng.randrange(129, 700), 16 * rng.randrange(9, 50), 16 * rng.randrange(16, 60)
        elif kind == "small":
            M, N, K = rng.randrange(1, 140), rng.randrange(1, 300), 16 * rng.randrange(1, 40)
        else:
            M, N, K = rng.randrange(1, 400), rng.randrange(1, 400), rng.randrange(1, 500)
        fa, fb = rng.choice([O.E4M3, O.E5M2]), rng.choice([O.E4M3, O.E5M2])
        bt = rng.random() < 0.5 and N % 16 == 0 and K % 16 == 0 and M > 128 and N > 128 and K >= 256
        at = bt and M % 16 == 0 and rng.random() < 0.5
        dd = rng.choice([nt.F32, nt.F32, nt.BF16, nt.F16, nt.OUT_E4M3, nt.OUT_E5M2])
        fp8o = dd in (nt.OUT_E4M3, nt.OUT_E5M2)
        if fp8o and bt and M % 4 != 0: bt = at = False
        acc = dd == nt.F32 and rng.random() < 0.4
        bias_dt = rng.choice([None, None, torch.float32, torch.bfloat16]) if not bt else None
        inv = rng.random() < 0.3
        integer = rng.random() < 0.4
        print(f"seed {seed} case {case}: {kind} M={M} N={N} K={K} fa={fa} fb={fb} bt={bt} at={at} d={dd} acc={acc} bias={bias_dt} inv={inv} int={integer}", flush=True)
        g = torch.Generator(device=dev).manual_seed(1000 * seed + case)
        def operand(rows, cols, fmt):
            if integer:
                vals = torch.randint(-3, 4, (rows, cols), generator=g, device=dev).float()
                scale = 1.0
            else:
                vals = torch.randn((rows, cols), generator=g, device=dev)
                scale = float(2.0 ** rng.randrange(-2, 5))
            q = torch.empty(rows, cols, dtype=torch.uint8, device=dev)
            sc = torch.tensor([scale], device=dev)
            nt.check(nt.lib.ntfp8_cast_to_fp8(vals.data_ptr(), nt.F32, rows, cols, sc.data_ptr(), 0 if fmt == O.E4M3 else 1, q.data_ptr(), None, st), "cast")
            return q, sc
        aq, sa = operand(M, K, fa)
        bq, sb = operand(N, K, fb)
        a64 = tabs[fa][aq.long()] / sa.double()
        b64 = tabs[fb][bq.long()] / sb.double()
        ref = a64 @ b64.t()
        bias = None
        if bias_dt is not None:
            bias = (torch.randint(-4, 5, (N,), generator=g, device=dev).float() if integer else torch.randn(N, generator=g, device=dev)).to(bias_dt)
            ref = ref + bias.double()
        a_dev = aq.t().contiguous() if at else aq
        b_dev = bq.t().contiguous() if bt else bq
        d = nt.GemmDesc()
        ssa, ssb = ((1.0 / sa), (1.0 / sb)) if inv else (sa, sb)
        d.A, d.scale_a, d.B, d.scale_b = a_dev.data_ptr(), ssa.data_ptr(), b_dev.data_ptr(), ssb.data_ptr()
        d.M, d.N, d.K, d.fmt_a, d.fmt_b = M, N, K, 0 if fa == O.E4M3 else 1, 0 if fb == O.E4M3 else 1
        d.b_transposed, d.a_transposed, d.scales_are_inverse = int(bt), int(at), int(inv)
        d.d_dtype, d.accumulate = dd, int(acc)
        if bias is not None: d.bias, d.bias_dtype = bias.data_ptr(), nt.TORCH_TO_NT[bias.dtype]
        if fp8o:
            out = torch.zeros(M, N, dtype=torch.uint8, device=dev)
            out_t = torch.zeros(N, M, dtype=torch.uint8, device=dev) if rng.random() < 0.5 else None
            sd = torch.tensor([float(2.0 ** rng.randrange(-3, 3))], device=dev)
            d.D, d.scale_d, d.D_t, d.amax_workspace = out.data_ptr(), sd.data_ptr(), nt.ptr(out_t), ws.data_ptr()
        else:
            prev = ((torch.randint(-50, 51, (M, N), generator=g, device=dev).float() if integer else torch.randn(M, N, generator=g, device=dev)).to(TD[dd])) if acc else None
            out = prev.clone() if acc else torch.full((M, N), 7.0, dtype=TD[dd], device=dev)
            d.D = out.data_ptr()
            if acc: ref = ref + prev.double()
        rc = nt.lib.ntfp8_gemm_batch((nt.GemmDesc * 1)(d), 1, st)
        if rc != 0:
            bad.append((case, "rc", rc))
            continue
        if fp8o:
            am = torch.zeros(1, device=dev); us = torch.zeros(1, device=dev)
            nt.check(nt.lib.ntfp8_amax_finalize(ws.data_ptr(), 0 if dd == nt.OUT_E4M3 else 1, 0, sd.data_ptr(), None, 0, am.data_ptr(), us.data_ptr(), st), "fin")
            torch.cuda.synchronize()
            fo = O.E4M3 if dd == nt.OUT_E4M3 else O.E5M2
            got = tabs[fo][out.long()] / sd.double()
            # compare against the cast of the library's own fp32 result (bit-exact) and the amax against it
            d2 = nt.GemmDesc.from_buffer_copy(d)
            hp = torch.empty(M, N, dtype=torch.float32, device=dev)
            d2.D, d2.d_dtype, d2.scale_d, d2.D_t, d2.amax_workspace = hp.data_ptr(), nt.F32, None, None, None
            nt.check(nt.lib.ntfp8_gemm_batch((nt.GemmDesc * 1)(d2), 1, st), "hp")
            q2 = torch.empty(M, N, dtype=torch.uint8, device=dev)
            nt.check(nt.lib.ntfp8_cast_to_fp8(hp.data_ptr(), nt.F32, M, N, sd.data_ptr(), 0 if fo == O.E4M3 else 1, q2.data_ptr(), None, st), "cast2")
            torch.cuda.synchronize()
            ok = torch.equal(out, q2) and (out_t is None or torch.equal(out_t, out.t().contiguous()))
            ok = ok and float(am) == float(hp.abs().max())
            rel = float((hp.double() - ref).norm() / ref.norm().clamp_min(1e-30))
            ok = ok and (rel <= 1e-3 if not integer else torch.equal(hp.double(), ref))
        else:
            torch.cuda.synchronize()
            if integer and dd == nt.F32:
                ok = torch.equal(out.double(), ref); rel = 0.0
            else:
                tol = 1e-3 if dd == nt.F32 else (4e-3 if dd == nt.BF16 else 1e-3)
                rel = float((out.double() - ref).norm() / ref.norm().clamp_min(1e-30))
                ok = rel <= tol
        if not ok:
            bad.append((case, kind, M, N, K, fa, fb, bt, at, dd, acc, str(bias_dt), inv, integer, rel))
    assert not bad, bad
