#!/usr/bin/env python3
"""Benchmark of the FP8 linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload linear|quant] [--no-cpu-baseline]

Default workload ("linear"): the Llama-3-8B decoder-block linears of the benchmark configuration,
forward + backward with delayed scaling (history 16, margin 0) at 4096 tokens:
QKV 4096->6144, O 4096->4096, gate 4096->14336, up 4096->14336, down 14336->4096.
One step = the bf16 master weights take the step's (perturbed) values and their fp8 copies are refreshed
(e4m3, one batched call); then for every linear: quantise the step's activation (e4m3), forward GEMM (bf16 out),
quantise the step's output gradient (e5m2, with its transposed copy), dgrad GEMM (bf16 out) and wgrad GEMM (fp32
out) in one batched call.  Inputs of ten steps (fresh seeded X / dY, perturbed weights) are resident in HBM before
the timed region and are walked round robin.  Before anything is timed, steps 0 and 1 are compared with the CPU
oracle (bit-exact amax / scales / histories / fp8 bytes, GEMM results within rel-L2 1e-3); a mismatch ends the run
without a line.  value = GEMM FLOPs of the step (6*M*N*K per linear) / wall time of the step, so the quantisation
passes are inside the time but contribute no FLOPs.

Workload "quant": benchmark configuration 2, the fused amax + history roll + scale update +
saturating cast on bf16 [4096,4096], e4m3 and e5m2 alternating, 8 rotating input buffers.

One JSON line is printed.  `roofline` describes the dominant kernel (the fp8 MFMA GEMM for
"linear", the fused quantise kernel for "quant"), timed with events on the launch stream;
`cpu_baseline` is the CPU oracle (a port of the reference's arithmetic) timed on this host.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0  # MI355X dense fp8 MFMA peak
PEAK_HBM_GBPS = 8000.0    # MI355X HBM3E peak
# HBM-side traffic is not measurable from inside this process: it comes from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# runs of this same script, whose summary (figures, commands, the commit and flags they were taken at) is the text
# file below.  Its "bench-readable" block is parsed here and handed on with its provenance.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic_counters.txt")

TOKENS = 4096
LINEARS = [  # name, in_features (K), out_features (N): benchmark configuration 5 (the parity test uses the same list)
    ("qkv", 4096, 6144),
    ("o", 4096, 4096),
    ("gate", 4096, 14336),
    ("up", 4096, 14336),
    ("down", 14336, 4096),
]


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=20)
    p.add_argument("--warmup", type=int, default=5)
    p.add_argument("--workload", choices=["linear", "quant", "probe", "vendor-gemm", "wg-timeline"], default="linear",
                   help="linear: the headline step; quant: configuration 2; probe: a few launches for counter runs; "
                        "vendor-gemm: hipBLASLt's fp8 GEMM next to this library's on the forward shapes")
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--weight-stream", action="store_true",
                   help="re-quantise the weights on a second stream (measured: no gain, the GEMMs are power-bound)")
    p.add_argument("--transposed-copies", action="store_true",
                   help="quantise weights and inputs together with transposed copies and run the backward GEMMs on "
                        "those (the reference's way) instead of letting the GEMM read the tensors as they are")
    p.add_argument("--grad-transposed-copy", action="store_true",
                   help="quantise the output gradient together with its transposed copy and run wgrad on that (the "
                        "reference's way, kernel.py:44) instead of letting the GEMM read dY as it is")
    p.add_argument("--kernel-reps", type=int, default=0,
                   help="also time each GEMM shape in isolation with this many back-to-back launches (0 = skip)")
    p.add_argument("--operand-sets", type=int, default=4,
                   help="vendor-gemm: operand sets walked round robin (1 = operands stay in the memory-side cache)")
    p.add_argument("--fp8-activations", action="store_true",
                   help="every linear returns its output as an e4m3 FP8Tensor quantised in the GEMM epilogue "
                        "(no bf16 activation is written); not the headline configuration")
    p.add_argument("--no-graph", action="store_true",
                   help="linear workload: launch every step from Python instead of replaying HIP graphs of the steps "
                        "(one graph per input set, captured after the correctness gate)")
    p.add_argument("--no-verify", action="store_true",
                   help="skip the correctness gate (profiling runs only: the line then says verified = false)")
    return p.parse_args()


def capture_steps(mods, sets, wstream, fp8_out):
    """One HIP graph per input set: the step is captured as the eager code issues it (same kernels, same order), the
    graphs share one memory pool and are replayed in capture order, round robin.  The scaling state lives outside the
    pool and carries over from replay to replay exactly as from eager step to eager step.  Every role must hold a scale
    already (a role's first quantisation reads its amax on the host)."""
    import torch

    assert all(st.initialised for lin in mods for st in lin.scaling.values()), "run two eager steps before capturing"
    graphs, pool = [], None
    for j in range(len(sets)):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, pool=pool):
            linear_step(mods, sets, j, wstream, fp8_out=fp8_out)
        pool = g.pool()
        graphs.append(g)
    return graphs


def flags_of(args):
    """The switches that change which kernels a step launches, as one string (recorded next to counter figures)."""
    on = [n for n in ("weight_stream", "transposed_copies", "grad_transposed_copy", "fp8_activations") if getattr(args, n)]
    return "default" if not on else ",".join(on)


def read_traffic(args):
    """{"gemm": bytes per step | None, "quant": bytes per launch | None, "source": {...}} from the bench-readable
    block of the counter summary under profiles/.  A figure taken with other flags than this run's is not used."""
    out = {"gemm": None, "quant": None, "source": {"file": os.path.relpath(TRAFFIC_FILE, ROOT)}}
    try:
        text = open(TRAFFIC_FILE).read()
    except OSError:
        out["source"]["note"] = "file not found"
        return out
    kv = {}
    block = False
    for line in text.splitlines():
        if line.startswith("[bench-readable]"):
            block = True
            continue
        if block and "=" in line:
            k, v = line.split("=", 1)
            kv[k.strip()] = v.strip()
    out["source"].update({"commit": kv.get("commit"), "flags": kv.get("flags"), "workload": kv.get("workload")})
    if kv.get("flags") != flags_of(args):
        out["source"]["note"] = f"counters were taken with flags '{kv.get('flags')}', this run uses '{flags_of(args)}': not used"
        return out
    try:
        out["gemm"] = float(kv["gemm_fetch_bytes_per_step"]) + float(kv["gemm_write_bytes_per_step"])
        out["quant"] = float(kv["quant_fetch_bytes_per_launch"]) + float(kv["quant_write_bytes_per_launch"])
    except (KeyError, ValueError):
        out["source"]["note"] = "bench-readable block incomplete"
    return out


def event_time_ms(fn, reps, warm=3):
    import torch

    for _ in range(warm):
        fn()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / reps


# ------------------------------------------------------------------------------------ package power
def _power_files():
    """(power1_input, power1_cap) of the first GPU's hwmon node, in microwatts; (None, None) where the driver exposes
    none.  These boxes have one GPU."""
    import glob

    for d in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*")):
        f = os.path.join(d, "power1_input")
        if os.access(f, os.R_OK):
            cap = os.path.join(d, "power1_cap")
            return f, cap if os.access(cap, os.R_OK) else None
    return None, None


def package_power(fn, seconds=1.0, period=0.004):
    """Package power while `fn(i)` is launched back to back for `seconds` (the queue is kept a few calls deep and
    never drains): a thread reads the driver's power sensor every `period` seconds; the first third of the samples
    (ramp-up, sensor averaging) is dropped.  Returns None where there is no sensor."""
    import threading

    import torch

    f, cap = _power_files()
    if f is None:
        return None
    samples, stop = [], threading.Event()

    def sampler():
        while not stop.is_set():
            try:
                samples.append(int(open(f).read()) * 1e-6)
            except (OSError, ValueError):
                pass
            time.sleep(period)

    for i in range(3):
        fn(i)
    torch.cuda.synchronize()
    th = threading.Thread(target=sampler, daemon=True)
    th.start()
    t0, i, events = time.perf_counter(), 0, []
    while time.perf_counter() - t0 < seconds:
        fn(i)
        i += 1
        ev = torch.cuda.Event()
        ev.record()
        events.append(ev)
        if len(events) > 8:
            events.pop(0).synchronize()
    torch.cuda.synchronize()
    stop.set()
    th.join()
    kept = samples[len(samples) // 3:]
    if not kept:
        return None
    out = {"watts_mean": round(sum(kept) / len(kept), 1), "watts_max": round(max(kept), 1), "samples": len(kept),
           "calls": i, "seconds": seconds, "sensor": "hwmon power1_input (package), read every %g ms" % (period * 1e3)}
    if cap is not None:
        try:
            out["cap_watts"] = round(int(open(cap).read()) * 1e-6, 1)
        except (OSError, ValueError):
            pass
    return out


# ------------------------------------------------------------------------------------ linear workload
def build_linears(device, nsets, fp8_out=False):
    """The five linears, and `nsets` steps' worth of inputs resident in HBM: per step and layer a fresh seeded X and
    dY (generated on the CPU, as the oracle sees them) and a version of the bf16 master weight, each version the
    previous one plus a seeded perturbation: the stand-in for an optimizer update, so that the weight role's amax
    history moves.  A step swaps the layer's parameter for that step's version (a pointer swap, no device work)."""
    import torch

    from nanotron_amd.fp8 import DTypes, FP8Linear, FP8Parameter
    from oracle import step_check as C

    mods, cpu = [], []
    sets = [{"x": [], "gy": [], "w": []} for _ in range(nsets)]
    for i, (name, K, N) in enumerate(LINEARS):
        lin = FP8Linear(K, N, bias=False, device=device, out_dtype=DTypes.FP8E4M3 if fp8_out else torch.bfloat16,
                        delayed_scaling=True, amax_history_len=16, margin=0)
        w = C.initial_weight(i, K, N)
        per_step = []
        for s_ in range(nsets):
            w = C.perturbed_weight(w, s_, i)
            x, gy = C.step_inputs(s_, i, K, N)
            sets[s_]["w"].append(FP8Parameter(w.to(device), DTypes.FP8E4M3))
            sets[s_]["x"].append(x.to(device).requires_grad_(True))
            sets[s_]["gy"].append(gy.to(device))
            if s_ < 2:   # what the correctness gate compares with
                per_step.append((x, w, gy))
        lin.weight = sets[0]["w"][i]
        lin.keep_quantised_grad = True   # the correctness gate compares the e5m2 bytes of dY too (switched off after it)
        mods.append(lin)
        cpu.append(per_step)
    return mods, sets, cpu


def linear_step(mods, sets, index, wstream=None, fp8_out=False, check=None):
    """One step: the master weights take this step's values, the fp8 copies of all weights are refreshed (one batched
    library call on the compute stream, or per layer on a second stream), then forward + backward of every linear.
    `check(i, lin, x, y, saved_input)` is called after each layer by the correctness gate."""
    from nanotron_amd.fp8.optim import requantize_fp8_weights

    cur = sets[index % len(sets)]
    for lin, w in zip(mods, cur["w"]):
        lin.weight = w
    requantize_fp8_weights(mods, stream=wstream)
    for i, (lin, x, gy) in enumerate(zip(mods, cur["x"], cur["gy"])):
        x.grad = None
        y = lin(x)
        saved = y.grad_fn.saved_tensors[0] if check is not None and y.grad_fn is not None else None
        if fp8_out:
            y._grad_handle.backward(gy)   # the gradient of an fp8 output travels through its handle
        else:
            y.backward(gy)
        if check is not None:
            check(i, lin, x, y, saved)


def verify_steps(mods, sets, cpu, wstream):
    """The correctness gate: steps 0 and 1 of the workload (the first quantises with current scaling, the second
    runs the fused delayed-scaling kernels that the timed steps run) are compared layer by layer with the CPU oracle:
    amax, scales, amax histories and fp8 bytes bit for bit, Y / dX / dW on sampled rows within rel-L2 1e-3.
    Raises AssertionError on the first difference.  Returns the largest rel-L2 seen per GEMM kind."""
    from oracle import step_check as C

    assert C.LINEARS == LINEARS and C.TOKENS == TOKENS
    refs = C.new_reference_state()
    worst = {"fwd": 0.0, "dgrad": 0.0, "wgrad": 0.0}
    for step in range(2):
        def check(i, lin, x, y, saved):
            xc, wc, gc = cpu[i][step]
            errs = C.check_layer(f"step {step} {LINEARS[i][0]}", lin, refs[i], xc, wc, gc, y.detach(), x.grad,
                                 lin.weight.main_grad, saved, step, i, gq_gpu=lin.quantised_grad_output)
            for k, v in errs.items():
                worst[k] = max(worst[k], v)
        linear_step(mods, sets, step, wstream, check=check)
    for lin in mods:
        lin.keep_quantised_grad, lin.quantised_grad_output = False, None
    return {k: float(f"{v:.3e}") for k, v in worst.items()}


def gemm_algorithmic_bytes():
    """Operand bytes read once plus output bytes written once, summed over the 15 GEMMs of a step
    (fp8 operands; bf16 outputs for forward and dgrad, fp32 for wgrad)."""
    T, total = TOKENS, 0
    for _, K, N in LINEARS:
        total += (T * K + N * K + 2 * T * N) + (T * N + N * K + 2 * T * K) + (T * N + T * K + 4 * N * K)
    return float(total)


def gemm_in_step_timing(step, first_index, steps):
    """Times every GEMM call where it runs: `steps` further steps of the same workload with a HIP event
    recorded on the launch stream before and after each call of the GEMM entry points (a backward issues
    its dgrad and wgrad as one batched call).  Returns (flops, milliseconds) summed over one step and the
    per-call averages in call order."""
    import torch

    from nanotron_amd.fp8 import kernel as K

    orig_one, orig_batch, orig_fp8 = K._gemm_nt, K._gemm_nt_batch, K._gemm_nt_fp8
    log = []

    def bracket(fn, shapes):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        out = fn()
        e1.record()
        log.append((shapes, e0, e1))
        return out

    def timed_one(a, b, out_dtype, accumulate_into, bias=None):
        return bracket(lambda: orig_one(a, b, out_dtype, accumulate_into, bias), [(a.shape[0], b.shape[0], a.shape[1])])

    def timed_fp8(a, b, dtype, state, with_transpose, bias=None, bt=False, at=False):
        mnk = (a.shape[1 if at else 0], b.shape[1 if bt else 0], a.shape[0 if at else 1])
        return bracket(lambda: orig_fp8(a, b, dtype, state, with_transpose, bias, bt, at), [mnk])

    def timed_batch(problems):
        # elements 5 and 7 of a problem mark operands handed over as their transposes ([K, N] / [K, M])
        def mnk(p):
            bt = len(p) > 4 and p[4]
            at = len(p) > 6 and p[6]
            return (p[0].shape[1 if at else 0], p[1].shape[1 if bt else 0], p[0].shape[0 if at else 1])
        return bracket(lambda: orig_batch(problems), [mnk(p) for p in problems])

    K._gemm_nt, K._gemm_nt_batch, K._gemm_nt_fp8 = timed_one, timed_batch, timed_fp8
    try:
        for i in range(steps):
            step(first_index + i)
        torch.cuda.synchronize()
    finally:
        K._gemm_nt, K._gemm_nt_batch, K._gemm_nt_fp8 = orig_one, orig_batch, orig_fp8
    per_step = len(log) // steps
    names = [f"{n}.{t}" for n, _, _ in LINEARS for t in ("fwd", "dgrad+wgrad")]
    assert per_step == len(names), (per_step, len(names))
    total_flops, total_ms, per_call = 0.0, 0.0, []
    for c in range(per_step):
        shapes = log[c][0]
        ms = sum(log[s * per_step + c][1].elapsed_time(log[s * per_step + c][2]) for s in range(steps)) / steps
        flops = sum(2.0 * M * N * Kd for M, N, Kd in shapes)
        total_flops += flops
        total_ms += ms
        per_call.append({"gemm": names[c], "mnk": [list(x) for x in shapes], "ms": round(ms, 4),
                         "tflops": round(flops / ms / 1e9, 1)})
    return total_flops, total_ms, per_call


def gemm_isolated_timing(mods, sets, reps):
    """Back-to-back launches of each GEMM of the step on fixed operands (which then sit in the 256 MB
    memory-side cache): an upper bound on what the kernel does in the step, reported for comparison."""
    import torch

    from nanotron_amd.fp8 import DTypes, FP8Tensor
    from nanotron_amd.fp8.kernel import _gemm_nt

    per_shape = []
    for (name, K, N), lin, x, gy in zip(LINEARS, mods, sets[0]["x"], sets[0]["gy"]):
        xq = FP8Tensor(x.detach(), DTypes.FP8E4M3, with_transpose=True)
        gq = FP8Tensor(gy, DTypes.FP8E5M2, with_transpose=True)
        wq = lin.weight.data
        calls = [
            ("fwd", lambda: _gemm_nt(xq, wq, torch.bfloat16, None)),
            ("dgrad", lambda: _gemm_nt(gq, wq.transposed(), torch.bfloat16, None)),
            ("wgrad", lambda: _gemm_nt(gq.transposed(), xq.transposed(), torch.float32, None)),
        ]
        flops = 2.0 * TOKENS * N * K
        for tag, fn in calls:
            ms = event_time_ms(fn, reps)
            per_shape.append({"gemm": f"{name}.{tag}", "ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 1)})
    return per_shape


def cpu_baseline_linear():
    """The oracle's arithmetic for one linear (the O projection, 4096x4096x4096) forward + backward
    on this host: amax/scale/cast of X, W, dY and the three fp32 GEMMs on exactly-upcast operands."""
    import torch

    from oracle import fp8_oracle as O

    torch.set_num_threads(os.cpu_count() or 1)
    M = K = N = 4096
    x = O.normal_tensor(1, (M, K), 1.0)
    w = O.normal_tensor(2, (N, K), 0.02)
    gy = O.normal_tensor(3, (M, N), 1e-3)

    def run():
        xq, wq, gq = O.quantise_current(x, O.E4M3), O.quantise_current(w, O.E4M3), O.quantise_current(gy, O.E5M2)
        y = O.linear_forward(xq, wq, torch.bfloat16)
        dx = O.linear_dgrad(gq, wq, torch.bfloat16)
        dw = O.linear_wgrad(gq, xq)
        return y, dx, dw

    run()
    t0 = time.perf_counter()
    n = 0
    while n < 2 or time.perf_counter() - t0 < 10.0:
        run()
        n += 1
    dt = (time.perf_counter() - t0) / n
    return {"value": round(6.0 * M * N * K / dt / 1e12, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "kind": "port", "sample": f"O projection 4096x4096x4096 fwd+bwd (quantise X,W,dY + 3 fp32 GEMMs), {n} runs",
            "reference_cpu_path": cpu_reference_path_config1()}


def cpu_reference_path_config1():
    """What the reference itself executes when the tensors are on the CPU: plain `F.linear` in the tensors' own
    precision, no FP8 at all (src/nanotron/fp8/linear.py:53-54), on benchmark configuration 1 (X [2048,1024] ~N(0,1),
    W [1024,1024] ~N(0,0.02)), fp32 as FP8Linear(device="cpu") creates its weight.  Forward only, as the configuration."""
    import torch
    import torch.nn.functional as F

    from oracle import fp8_oracle as O

    x = O.normal_tensor(1234 + 100, (2048, 1024), 1.0, torch.float32)
    w = O.normal_tensor(1234 + 101, (1024, 1024), 0.02, torch.float32)
    for _ in range(3):
        F.linear(x, w)
    times = []
    t_end = time.perf_counter() + 3.0
    while len(times) < 5 or time.perf_counter() < t_end:
        t0 = time.perf_counter()
        F.linear(x, w)
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    return {"value": round(2.0 * 2048 * 1024 * 1024 / med / 1e12, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "kind": "reference", "sample": f"config 1: fp32 F.linear X[2048,1024] . W[1024,1024]^T on the CPU, median of {len(times)} runs"}


# ------------------------------------------------------------------------------------ quant workload
def build_quant(device, nbuf=8):
    import torch

    from nanotron_amd.fp8 import DelayedScaling, DTypes
    from oracle import fp8_oracle as O

    bufs = [O.student_t_outlier_tensor(1234 + 200 + i, (4096, 4096)).to(device) for i in range(nbuf)]
    states = {DTypes.FP8E4M3: DelayedScaling(DTypes.FP8E4M3, 16, 0, device),
              DTypes.FP8E5M2: DelayedScaling(DTypes.FP8E5M2, 16, 0, device)}
    return bufs, states


def quant_step(bufs, states, i):
    from nanotron_amd.fp8 import FP8Tensor

    x = bufs[i % len(bufs)]
    for dt, st in states.items():
        FP8Tensor(x, dt, state=st)


def quant_kernel_ms(bufs, states, reps):
    """Average duration of the fused delayed-scaling kernel alone (C ABI, preallocated outputs)."""
    import torch

    from nanotron_amd import _native as nt
    from nanotron_amd.fp8 import DTypes

    dev = bufs[0].device
    rows, cols = bufs[0].shape
    out = [torch.empty(rows * cols, dtype=torch.uint8, device=dev) for _ in range(len(bufs))]
    sc = torch.zeros(2, dtype=torch.float32, device=dev)
    ws = nt.workspace(dev)
    st = nt.stream_ptr(dev)
    res = {}
    for dt, fmt in ((DTypes.FP8E4M3, nt.E4M3), (DTypes.FP8E5M2, nt.E5M2)):
        state = states[dt]
        k = [0]

        def fn():
            i = k[0] % len(bufs)
            k[0] += 1
            nt.check(nt.lib.ntfp8_quantize_delayed(bufs[i].data_ptr(), nt.BF16, rows, cols, fmt, 0,
                                                   state.scale.data_ptr(), state.amax_history.data_ptr(), 16,
                                                   sc[0:].data_ptr(), sc[1:].data_ptr(), out[i].data_ptr(), None,
                                                   ws.data_ptr(), st), "quantize_delayed")

        res[dt.name] = event_time_ms(fn, reps, warm=8)
    return res


def quant_dual_kernel_ms(bufs, states, reps):
    """Average duration of the kernel that produces both formats from one pass over the tensor."""
    import torch

    from nanotron_amd import _native as nt
    from nanotron_amd.fp8 import DTypes

    dev = bufs[0].device
    n = bufs[0].numel()
    out4 = [torch.empty(n, dtype=torch.uint8, device=dev) for _ in range(len(bufs))]
    out5 = [torch.empty(n, dtype=torch.uint8, device=dev) for _ in range(len(bufs))]
    sc = torch.zeros(3, dtype=torch.float32, device=dev)
    ws = nt.workspace(dev)
    st = nt.stream_ptr(dev)
    s4, s5 = states[DTypes.FP8E4M3], states[DTypes.FP8E5M2]
    k = [0]

    def fn():
        i = k[0] % len(bufs)
        k[0] += 1
        nt.check(nt.lib.ntfp8_quantize_delayed_dual(bufs[i].data_ptr(), nt.BF16, n, 0, s4.scale.data_ptr(),
                                                    s4.amax_history.data_ptr(), s5.scale.data_ptr(), s5.amax_history.data_ptr(),
                                                    16, sc.data_ptr(), sc.data_ptr() + 4, sc.data_ptr() + 8,
                                                    out4[i].data_ptr(), out5[i].data_ptr(), ws.data_ptr(), st), "quantize_delayed_dual")

    return event_time_ms(fn, reps, warm=8)


def stream_probe_ms(bufs, reps):
    """The bandwidth yardsticks of the library (ntfp8_stream_probe: the flat quantise kernel's grid and access pattern
    without its arithmetic and reduction) on the same rotating tensors: read-only, 2 bytes read per byte written (the
    traffic of a bf16 -> fp8 cast), copy.  Milliseconds per launch."""
    import torch

    from nanotron_amd import _native as nt

    dev = bufs[0].device
    nbytes = bufs[0].numel() * bufs[0].element_size()
    dst = [torch.empty(nbytes, dtype=torch.uint8, device=dev) for _ in range(2)]
    st = nt.stream_ptr(dev)
    res = {}
    for name, mode in (("read_only", 0), ("read_2B_write_1B", 1), ("copy", 2)):
        k = [0]

        def fn():
            i = k[0]
            k[0] += 1
            nt.check(nt.lib.ntfp8_stream_probe(mode, bufs[i % len(bufs)].data_ptr(), nbytes, dst[i % 2].data_ptr(), st),
                     "ntfp8_stream_probe")

        res[name] = event_time_ms(fn, reps, warm=8)
    # the same copy by the vendor's kernel (torch's copy_ of a contiguous tensor), for scale
    views = [b.view(torch.uint8).reshape(-1) for b in bufs]
    k = [0]

    def vcopy():
        i = k[0]
        k[0] += 1
        dst[i % 2].copy_(views[i % len(views)])

    res["copy_by_torch"] = event_time_ms(vcopy, reps, warm=8)
    return res


def quant_report(device, traffic):
    """The `quant` object of the JSON line: the fused quantise kernel on benchmark configuration 2 (bf16 [4096,4096],
    8 rotating buffers so that the input does not sit in the memory-side cache), the both-formats-in-one-pass kernel on
    the same tensor, and the single-format kernel on the largest tensors of the step, where the launch ramp and the
    end-of-kernel reduction weigh less."""
    import torch

    from nanotron_amd.fp8 import DelayedScaling, DTypes

    bufs, states = build_quant(device)
    for i in range(2):   # both roles hold a scale from here on
        quant_step(bufs, states, i)
    qms = quant_kernel_ms(bufs, states, 64)
    qb = 3.0 * 4096 * 4096
    q_avg = sum(qms.values()) / len(qms)
    dual_ms = quant_dual_kernel_ms(bufs, states, 64)
    probe = stream_probe_ms(bufs, 64)
    rep = {"metric": "amax+quant GB/s", "value": round(qb / (q_avg * 1e-3) / 1e9, 1), "unit": "GB/s",
           "workload": "bf16 [4096,4096] fused amax+roll+scale+cast, 8 rotating buffers",
           "ms": {k: round(v, 5) for k, v in qms.items()},
           "roofline": {"bound": "hbm", "achieved": round(qb / (q_avg * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                        "frac": round(qb / (q_avg * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4), "traffic": traffic["quant"],
                        "algorithmic_bytes": qb, "kernel": "quant_flat_kernel",
                        "frac_of_yardstick": round(probe["read_2B_write_1B"] / q_avg, 4)},
           "yardstick": {"what": "ntfp8_stream_probe on the same tensors: same grid and 128-bit streaming accesses, no arithmetic, "
                                 "no reduction; copy_by_torch: the same copy by torch's copy_",
                         **{k: {"ms": round(v, 5), "GBps": round(b * 4096 * 4096 / (v * 1e-3) / 1e9, 1)}
                            for (k, v), b in zip(probe.items(), (2.0, 3.0, 4.0, 4.0))}},
           "both_formats_one_pass": {"ms": round(dual_ms, 5), "algorithmic_bytes": 4.0 * 4096 * 4096,
                                     "GBps": round(4.0 * 4096 * 4096 / (dual_ms * 1e-3) / 1e9, 1),
                                     "frac": round(4.0 * 4096 * 4096 / (dual_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4),
                                     "kernel": "quant_flat_dual_kernel"}}
    del bufs
    large = {}
    g = torch.Generator(device=device).manual_seed(99)
    for shape in ((4096, 14336), (14336, 4096)):
        lb = [torch.randn(shape, generator=g, device=device, dtype=torch.float32).to(torch.bfloat16) for _ in range(4)]
        st = {DTypes.FP8E4M3: DelayedScaling(DTypes.FP8E4M3, 16, 0, device), DTypes.FP8E5M2: DelayedScaling(DTypes.FP8E5M2, 16, 0, device)}
        for i in range(2):
            quant_step(lb, st, i)
        ms = quant_kernel_ms(lb, st, 32)
        avg = sum(ms.values()) / len(ms)
        nbytes = 3.0 * shape[0] * shape[1]
        pr = stream_probe_ms(lb, 32)
        large[f"{shape[0]}x{shape[1]}"] = {"ms": round(avg, 5), "GBps": round(nbytes / (avg * 1e-3) / 1e9, 1),
                                            "frac": round(nbytes / (avg * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4),
                                            "yardstick_read_2B_write_1B_ms": round(pr["read_2B_write_1B"], 5),
                                            "yardstick_read_only_GBps": round(2.0 * shape[0] * shape[1] / (pr["read_only"] * 1e-3) / 1e9, 1),
                                            "yardstick_copy_GBps": round(4.0 * shape[0] * shape[1] / (pr["copy"] * 1e-3) / 1e9, 1),
                                            "copy_by_torch_GBps": round(4.0 * shape[0] * shape[1] / (pr["copy_by_torch"] * 1e-3) / 1e9, 1),
                                            "frac_of_yardstick": round(pr["read_2B_write_1B"] / avg, 4)}
        del lb
    rep["large_tensors"] = large
    return rep


def cpu_baseline_quant():
    import torch

    from oracle import fp8_oracle as O

    torch.set_num_threads(os.cpu_count() or 1)
    x = O.student_t_outlier_tensor(1234 + 200, (4096, 4096))
    sts = [O.DelayedScaling(O.E4M3), O.DelayedScaling(O.E5M2)]
    for s in sts:
        s.quantise(x)
    t0 = time.perf_counter()
    n = 0
    while n < 2 or time.perf_counter() - t0 < 10.0:
        for s in sts:
            s.quantise(x)
        n += 1
    dt = (time.perf_counter() - t0) / (2 * n)
    return {"value": round(3.0 * x.numel() / dt / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(),
            "kind": "port", "sample": f"bf16 [4096,4096] delayed-scaling quantise (amax, cast, roll), {2 * n} tensor-steps"}


# ------------------------------------------------------------------------------------ counter probe
def probe(device):
    """A handful of launches for `rocprofv3 --pmc` runs, in this order: one plain copy of known size (the
    calibration for FETCH_SIZE / WRITE_SIZE), the fused quantise kernels on the benchmark tensor (single format,
    both formats), and for the O-projection and gate shapes the three GEMMs as FP8Linear issues them: forward, then
    dgrad + wgrad in one batched call with W, X and dY read untransposed.  Prints what was launched."""
    import torch

    from nanotron_amd.fp8 import DTypes, FP8Tensor
    from nanotron_amd.fp8.kernel import _gemm_nt, _gemm_nt_batch

    src = torch.empty(128 * 1024 * 1024, dtype=torch.uint8, device=device).fill_(1)
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    dst.copy_(src)  # 128 MiB read + 128 MiB written
    bufs, states = build_quant(device, nbuf=2)
    for i in range(3):
        quant_step(bufs, states, i)
    quant_dual_kernel_ms(bufs, states, 2)
    g = torch.Generator(device="cpu").manual_seed(7)
    launched = {"copy": {"read_bytes": src.numel(), "write_bytes": src.numel()},
                "quant_flat_kernel": {"elements": 4096 * 4096, "algorithmic_bytes": 3 * 4096 * 4096},
                "quant_flat_dual_kernel": {"elements": 4096 * 4096, "algorithmic_bytes": 4 * 4096 * 4096}}
    for name, K, N in (("o", 4096, 4096), ("gate", 4096, 14336)):
        x = torch.randn(TOKENS, K, generator=g).to(torch.bfloat16).to(device)
        w = (torch.randn(N, K, generator=g) * 0.02).to(device)
        gy = (torch.randn(TOKENS, N, generator=g) * 1e-3).to(torch.bfloat16).to(device)
        xq, wq, gq = FP8Tensor(x, DTypes.FP8E4M3), FP8Tensor(w, DTypes.FP8E4M3), FP8Tensor(gy, DTypes.FP8E5M2)
        _gemm_nt(xq, wq, torch.bfloat16, None)
        _gemm_nt_batch([(gq, wq, torch.bfloat16, None, True), (gq, xq, torch.float32, None, True, None, True)])
        launched[f"gemm_{name}"] = {"M": TOKENS, "N": N, "K": K,
                                    "algorithmic_bytes_fwd": TOKENS * K + N * K + 2 * TOKENS * N,
                                    "algorithmic_bytes_dgrad": TOKENS * N + N * K + 2 * TOKENS * K,
                                    "algorithmic_bytes_wgrad": TOKENS * N + TOKENS * K + 4 * N * K}
    torch.cuda.synchronize()
    print(json.dumps({"probe": launched}))


# ------------------------------------------------------------------------------------ vendor library, for comparison
def _profiling_lib(path):
    """A profiling build of the library (nanotron_amd/profiling/, `python -m nanotron_amd.build --profiling`)."""
    import ctypes

    from nanotron_amd import _native as nt

    if not os.path.exists(path):
        raise FileNotFoundError(f"{path}: build it with `python -m nanotron_amd.build --profiling`")
    lib = ctypes.CDLL(path)
    lib.ntfp8_gemm_batch.restype = ctypes.c_int
    lib.ntfp8_gemm_batch.argtypes = [ctypes.POINTER(nt.GemmDesc), ctypes.c_int, ctypes.c_void_p]
    lib.ntfp8_debug_stamps.restype = ctypes.c_int
    lib.ntfp8_debug_stamps.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
    lib.ntfp8_debug_set_tile_order.restype = ctypes.c_int
    lib.ntfp8_debug_set_tile_order.argtypes = [ctypes.c_int]
    return lib


def _run_gemms(lib, probs, st):
    """One ntfp8_gemm_batch call of `lib`; a problem is (a, b, out, b_transposed, a_transposed, d_dtype)."""
    from nanotron_amd import _native as nt
    from nanotron_amd.fp8 import DTypes

    d = (nt.GemmDesc * len(probs))()
    for e, (a, b, out, bt, at, dd) in zip(d, probs):
        e.A, e.scale_a, e.B, e.scale_b, e.D = (a.data_ptr(), a.fp8_meta.scale.data_ptr(), b.data_ptr(),
                                               b.fp8_meta.scale.data_ptr(), out.data_ptr())
        (e.K, e.M) = a.shape if at else a.shape[::-1]
        e.N = b.shape[1] if bt else b.shape[0]
        e.fmt_a = 0 if a.fp8_meta.dtype == DTypes.FP8E4M3 else 1
        e.fmt_b = 0 if b.fp8_meta.dtype == DTypes.FP8E4M3 else 1
        e.d_dtype, e.accumulate, e.b_transposed, e.a_transposed = dd, 0, int(bt), int(at)
    rc = lib.ntfp8_gemm_batch(d, len(probs), st)
    assert rc == 0, rc


def _pcts(v):
    import numpy as np

    return {k: round(float(np.percentile(v, p)), 2) for k, p in (("p10", 10), ("p50", 50), ("p90", 90), ("max", 100))}


def _stamp_report(lib, n, k_tiles):
    """Phases of the `n` workgroups of the last big-kernel launch of `lib`, from the stamps they left."""
    import numpy as np

    pcts = _pcts
    buf = np.zeros(n * 8, dtype=np.uint64)
    rc = lib.ntfp8_debug_stamps(buf.ctypes.data, buf.nbytes)
    assert rc == 0, rc
    s = buf.reshape(n, 8).astype(np.int64)
    t = s[:, :5] * 0.01   # 100 MHz ticks -> us
    t0, t_end = t[:, 0].min(), t[:, 4].max()
    hw, xcc = s[:, 5] & 0xFFFFFFFF, (s[:, 5] >> 32) & 0xF
    cycles = (s[:, 7] - s[:, 6]).astype(np.float64)   # shader-clock cycles of the K loop
    cu = (xcc << 16) | (((hw >> 13) & 7) << 8) | (((hw >> 12) & 1) << 4) | ((hw >> 8) & 0xF)
    ids = np.unique(cu)
    handover, idle_end, per_cu = [], [], []
    for c in ids:
        idx = np.where(cu == c)[0]
        idx = idx[np.argsort(t[idx, 0])]
        per_cu.append(len(idx))
        idle_end.append(t_end - t[idx[-1], 4])
        handover += [t[b, 0] - t[a, 4] for a, b in zip(idx, idx[1:])]
    loop = t[:, 2] - t[:, 1]
    out = {"workgroups": n, "span_us": round(float(t_end - t0), 1), "cus": int(len(ids)),
           "workgroups_per_cu": [int(min(per_cu)), int(max(per_cu))],
           "us_per_workgroup": {"entry_to_first_tile": pcts(t[:, 1] - t[:, 0]), "k_loop": pcts(loop),
                                "epilogue_issue": pcts(t[:, 3] - t[:, 2]), "store_drain": pcts(t[:, 4] - t[:, 3]),
                                "whole": pcts(t[:, 4] - t[:, 0])},
           "k_loop_cycles_per_k_tile_p50": round(float(np.median(cycles)) / k_tiles, 1),
           "k_loop_us_per_k_tile_p50": round(float(np.median(loop)) / k_tiles, 3),
           "k_loop_shader_clock_ghz_p50": round(float(np.median(cycles / (loop * 1e3))), 3),
           "cu_idle_before_launch_end_us": pcts(idle_end),
           "k_loop_p50_by_xcd_us": [round(float(np.median(loop[xcc == k])), 1) for k in range(8)],
           "last_store_p50_by_xcd_us": [round(float(np.median([t[np.where(cu == c)[0], 4].max() - t0
                                                               for c in ids if (c >> 16) == k])), 1) for k in range(8)]}
    if handover:
        out["handover_on_a_cu_us"] = pcts(handover)
    return out


def loop_experiments(device, reps=3, launches=24):
    """What the K loop of a whole tile pays for, piece by piece, under sustained load: the experiment builds of the
    profiling library (nanotron_amd/build.py: EXPERIMENTS; parts of the loop left out, or idle cycles put in) run the
    one-round forward GEMMs of the O projection (K = 4096) and of the down projection (K = 14336) `launches` times
    back to back on rotating operand sets, alternating between the builds.  Per build: microseconds per launch (HIP
    events, best of `reps`), and from the stamps of the last launch the cycles per K-tile and the shader clock."""
    import torch

    from nanotron_amd import _native as nt
    from nanotron_amd.build import EXPERIMENTS, experiment_lib
    from nanotron_amd.fp8 import DTypes, FP8Tensor

    libs = [(name, _profiling_lib(experiment_lib(name))) for name in EXPERIMENTS]
    g = torch.Generator(device=device).manual_seed(5)
    st = nt.stream_ptr(device)
    bf16 = nt.TORCH_TO_NT[torch.bfloat16]
    out = {}
    for tag, K, nsets in (("o fwd 4096x4096x4096", 4096, 8), ("down fwd 4096x4096x14336", 14336, 4)):
        sets = []
        for _ in range(nsets):
            x = FP8Tensor(torch.randn(TOKENS, K, generator=g, device=device).to(torch.bfloat16), DTypes.FP8E4M3)
            w = FP8Tensor((torch.randn(4096, K, generator=g, device=device) * 0.02).to(torch.bfloat16), DTypes.FP8E4M3)
            sets.append((x, w, torch.empty(TOKENS, 4096, dtype=torch.bfloat16, device=device)))
        res = {name: {"us": []} for name, _ in libs}
        vendor = "hipblaslt (vendor kernel, same operands, no stamps)"
        res[vendor] = {"us": []}
        one = torch.tensor(1.0, device=device)
        views = [(x.as_subclass(torch.Tensor).view(torch.float8_e4m3fn), w.as_subclass(torch.Tensor).view(torch.float8_e4m3fn))
                 for x, w, _ in sets]
        for _ in range(reps):
            kv = [0]

            def vfn():
                a, b = views[kv[0] % nsets]
                kv[0] += 1
                torch._scaled_mm(a, b.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)

            res[vendor]["us"].append(round(event_time_ms(vfn, launches, warm=4) * 1e3, 1))
            for name, lib in libs:
                k = [0]

                def fn():
                    x, w, y = sets[k[0] % nsets]
                    k[0] += 1
                    _run_gemms(lib, [(x, w, y, False, False, bf16)], st)

                res[name]["us"].append(round(event_time_ms(fn, launches, warm=4) * 1e3, 1))
                rep = _stamp_report(lib, 256, K // 128)
                res[name].update({"cycles_per_k_tile": rep["k_loop_cycles_per_k_tile_p50"],
                                  "clock_ghz": rep["k_loop_shader_clock_ghz_p50"]})
        # package power of every build under the same sustained launches (a pass of its own, about a second each)
        kp = [0]

        def vpow(i):
            a, b = views[i % nsets]
            torch._scaled_mm(a, b.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)

        pw = package_power(vpow, seconds=0.8)
        if pw is not None:
            res[vendor]["watts"] = pw["watts_mean"]
        for name, lib in libs:
            def pfn(i, lib=lib):
                x, w, y = sets[i % nsets]
                _run_gemms(lib, [(x, w, y, False, False, bf16)], st)

            pw = package_power(pfn, seconds=0.8)
            if pw is not None:
                res[name]["watts"] = pw["watts_mean"]
                out["power_cap_watts"] = pw.get("cap_watts")
        # the kernel as it is on all-zero operands: same instructions, same cycles; what the matrix cores draw depends
        # on the operand bytes, so this shows how fast the schedule runs when power does not hold the clock down
        base_lib = dict(libs)["base"]
        zx = FP8Tensor(torch.zeros(TOKENS, K, dtype=torch.bfloat16, device=device), DTypes.FP8E4M3)
        zw = FP8Tensor(torch.zeros(4096, K, dtype=torch.bfloat16, device=device), DTypes.FP8E4M3)
        zy = sets[0][2]

        def zfn(i=0):
            _run_gemms(base_lib, [(zx, zw, zy, False, False, bf16)], st)

        zname = "base_zero_operands"
        res[zname] = {"us": [round(event_time_ms(zfn, launches, warm=4) * 1e3, 1) for _ in range(reps)]}
        rep = _stamp_report(base_lib, 256, K // 128)
        res[zname].update({"cycles_per_k_tile": rep["k_loop_cycles_per_k_tile_p50"], "clock_ghz": rep["k_loop_shader_clock_ghz_p50"]})
        pw = package_power(zfn, seconds=0.8)
        if pw is not None:
            res[zname]["watts"] = pw["watts_mean"]
        for name in res:
            res[name]["us_best"] = min(res[name]["us"])
            res[name]["tflops"] = round(2.0 * TOKENS * 4096 * K / res[name]["us_best"] / 1e6, 1)
        out[tag] = res
        del sets
    return out


def workgroup_timeline(device):
    """Where a workgroup of the GEMM kernel spends its time, read from the kernel itself: the profiling build of the
    library (nanotron_amd/profiling/libntfp8_stamps.so, -DNTFP8_STAMPS) stamps the 100 MHz wall clock five times per
    workgroup and records the CU it ran on.  Four launches without a half-tile tail: one round at K = 4096 and at
    K = 14336, three rounds, and the seven-round dgrad + wgrad launch of the down projection."""
    import torch

    from nanotron_amd import _native as nt
    from nanotron_amd.build import LIB_STAMPS
    from nanotron_amd.fp8 import DTypes, FP8Tensor

    lib = _profiling_lib(LIB_STAMPS)
    g = torch.Generator(device=device).manual_seed(1)

    def q(shape, std, dt):
        return FP8Tensor((torch.randn(shape, generator=g, device=device) * std).to(torch.bfloat16), dt)

    st = nt.stream_ptr(device)

    def run(probs):
        _run_gemms(lib, probs, st)

    def report(n, k_tiles):
        return _stamp_report(lib, n, k_tiles)

    T = TOKENS
    x, w = q((T, 4096), 1.0, DTypes.FP8E4M3), q((4096, 4096), 0.02, DTypes.FP8E4M3)
    w3 = q((12288, 4096), 0.02, DTypes.FP8E4M3)
    xd, wd = q((T, 14336), 1.0, DTypes.FP8E4M3), q((4096, 14336), 0.02, DTypes.FP8E4M3)
    gd = q((T, 4096), 1e-3, DTypes.FP8E5M2)
    y = torch.empty(T, 4096, dtype=torch.bfloat16, device=device)
    y3 = torch.empty(T, 12288, dtype=torch.bfloat16, device=device)
    dx = torch.empty(T, 14336, dtype=torch.bfloat16, device=device)
    dw = torch.empty(4096, 14336, dtype=torch.float32, device=device)
    bf16, f32 = nt.TORCH_TO_NT[torch.bfloat16], nt.TORCH_TO_NT[torch.float32]
    pair = [(gd, wd, dx, True, False, bf16), (gd, xd, dw, True, True, f32)]
    cases = [("o fwd 4096x4096x4096 -> bf16, 1 round", [(x, w, y, False, False, bf16)], 256, 32),
             ("fwd 4096x12288x4096 -> bf16, 3 rounds", [(x, w3, y3, False, False, bf16)], 768, 32),
             ("down fwd 4096x4096x14336 -> bf16, 1 round", [(xd, wd, y, False, False, bf16)], 256, 112),
             ("down dgrad (bf16) + wgrad (fp32), operands read untransposed, 7 rounds", pair, 1792, 32)]
    wh = q((2048, 4096), 0.02, DTypes.FP8E4M3)
    yh = torch.empty(T, 2048, dtype=torch.bfloat16, device=device)
    cases.append(("fwd 4096x2048x4096 -> bf16, 128 tiles as 256 half tiles (the tail kernel alone)",
                  [(x, wh, yh, False, False, bf16)], 256, 32))
    res = {}
    for tag, probs, n, kt in cases:
        for _ in range(6):
            run(probs)
        torch.cuda.synchronize()
        run(probs)
        torch.cuda.synchronize()
        res[tag] = report(n, kt)
    # what the fetch traffic costs: the same launches with the XCD-aware tile order switched off (every XCD then pulls
    # every operand panel through its own L2)
    for tag, probs, n, kt in cases[1:3]:
        for plain in (1, 0):
            assert lib.ntfp8_debug_set_tile_order(plain) == 0
            for _ in range(6):
                run(probs)
            torch.cuda.synchronize()
            run(probs)
            torch.cuda.synchronize()
            res[tag + (" | tiles in launch order" if plain else " | XCD-aware order (repeat)")] = report(n, kt)
    # the same seven-round launch on a rested chip and under sustained load
    torch.cuda.synchronize()
    time.sleep(0.3)
    run(pair)
    torch.cuda.synchronize()
    res["7-round launch, single, after 0.3 s of idle"] = report(1792, 32)
    for reps in (4, 16):
        for _ in range(reps):
            run(pair)
        torch.cuda.synchronize()
        res[f"7-round launch, last of {reps} back to back"] = report(1792, 32)
        time.sleep(0.3)
    return res


def hipblaslt_reference(device, reps=30, nsets=4):
    """The vendor's fp8 GEMM (hipBLASLt behind torch._scaled_mm, e4m3 x e4m3, bf16 output) on the forward shapes of
    the workload, rotating operands as the step does.  A yardstick for the hand-written kernel, not part of the
    product: nothing in nanotron_amd calls it."""
    import torch

    g = torch.Generator(device=device).manual_seed(3)
    one = torch.tensor(1.0, device=device)
    out = []
    for name, K, N in LINEARS:
        ops = []
        for _ in range(nsets):
            a = (torch.randn(TOKENS, K, generator=g, device=device) * 64).clamp(-448, 448).to(torch.float8_e4m3fn)
            b = (torch.randn(N, K, generator=g, device=device) * 64).clamp(-448, 448).to(torch.float8_e4m3fn)
            ops.append((a, b))
        k = [0]

        def fn():
            a, b = ops[k[0] % len(ops)]
            k[0] += 1
            return torch._scaled_mm(a, b.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)

        ms = event_time_ms(fn, reps, warm=6)
        out.append({"gemm": f"{name}.fwd", "mnk": [TOKENS, N, K], "ms": round(ms, 4),
                    "tflops": round(2.0 * TOKENS * N * K / ms / 1e9, 1)})
        del ops
    return out


def own_forward_reference(device, reps=30, nsets=4):
    """The same shapes, same rotation, through this library's forward GEMM (C ABI, outputs allocated beforehand, as
    torch does for the vendor call from its caching allocator)."""
    import torch

    from nanotron_amd import _native as nt
    from nanotron_amd.fp8 import DTypes, FP8Tensor

    g = torch.Generator(device=device).manual_seed(3)
    st = nt.stream_ptr(device)
    out = []
    for name, K, N in LINEARS:
        ops = []
        for _ in range(nsets):
            a = FP8Tensor(torch.randn(TOKENS, K, generator=g, device=device).to(torch.bfloat16), DTypes.FP8E4M3)
            b = FP8Tensor(torch.randn(N, K, generator=g, device=device).to(torch.bfloat16), DTypes.FP8E4M3)
            ops.append((a, b, torch.empty(TOKENS, N, dtype=torch.bfloat16, device=device)))
        k = [0]

        def fn():
            a, b, d = ops[k[0] % len(ops)]
            k[0] += 1
            nt.check(nt.lib.ntfp8_gemm(a.data_ptr(), nt.E4M3, a.fp8_meta.scale.data_ptr(), b.data_ptr(), nt.E4M3,
                                       b.fp8_meta.scale.data_ptr(), d.data_ptr(), nt.BF16, TOKENS, N, K, 0, st), "ntfp8_gemm")

        ms = event_time_ms(fn, reps, warm=6)
        out.append({"gemm": f"{name}.fwd", "mnk": [TOKENS, N, K], "ms": round(ms, 4),
                    "tflops": round(2.0 * TOKENS * N * K / ms / 1e9, 1)})
        del ops
    return out


# ------------------------------------------------------------------------------------ main
def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this hot path has no collectives and every box here has one GPU; "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (cuda:0)", file=sys.stderr)
        sys.exit(2)
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)
    if args.transposed_copies:
        import nanotron_amd.fp8.kernel as K

        K.READ_B_TRANSPOSED = False
    if args.grad_transposed_copy:
        import nanotron_amd.fp8.kernel as K

        K.READ_A_TRANSPOSED = False

    if args.workload == "probe":
        probe(device)
        return
    if args.workload == "wg-timeline":
        print(json.dumps({"workload": "per-workgroup wall-clock stamps inside gemm_nt_big_kernel (profiling builds)",
                          "launches": workgroup_timeline(device), "k_loop_experiments": loop_experiments(device)}))
        return
    if args.workload == "vendor-gemm":
        n = args.operand_sets
        print(json.dumps({"workload": f"forward GEMMs of the step, e4m3 x e4m3 -> bf16, {n} rotating operand set(s)",
                          "hipblaslt_scaled_mm": hipblaslt_reference(device, nsets=n),
                          "ntfp8": own_forward_reference(device, nsets=n)}))
        return
    traffic = read_traffic(args)
    verified = None
    if args.workload == "linear":
        # ten steps' worth of inputs (benchmark configuration 5), fewer if the run is shorter than that
        nsets = max(2, min(10, args.warmup + 2 * args.steps))
        mods, sets, cpu = build_linears(device, nsets, fp8_out=args.fp8_activations)
        wstream = torch.cuda.Stream(device=device) if args.weight_stream else None
        eager_step = lambda i: linear_step(mods, sets, i, wstream, fp8_out=args.fp8_activations)
        step = eager_step
        flops_step = sum(6.0 * TOKENS * N * K for _, K, N in LINEARS)
        first = 0
        if not args.no_verify and not args.fp8_activations:
            # correctness gate: no line is printed for a step that does not match the oracle
            try:
                verified = verify_steps(mods, sets, cpu, wstream)
            except AssertionError as e:
                print(f"bench.py: the workload's results differ from the CPU oracle, nothing measured: {e}", file=sys.stderr)
                sys.exit(1)
            first = 2
        del cpu
        for lin in mods:   # (only the gate looks at the quantised output gradient)
            lin.keep_quantised_grad, lin.quantised_grad_output = False, None
        graph_note = None
        if not args.no_graph:
            # two eager steps (the gate's, or these) have given every scaling role its first scale
            for i in range(first, 2):
                eager_step(i)
            first = max(first, 2)
            try:
                graphs = capture_steps(mods, sets, wstream, args.fp8_activations)
                step = lambda i: graphs[i % len(graphs)].replay()
            except Exception as e:   # reported, not hidden: the line then says the steps were launched eagerly
                graph_note = f"graph capture failed, eager launches instead: {type(e).__name__}: {e}"
                torch.cuda.synchronize()
    else:
        bufs, states = build_quant(device)
        step = lambda i: quant_step(bufs, states, i)
        bytes_step = 2 * 3.0 * 4096 * 4096
        first = 0

    for i in range(args.warmup):
        step(first + i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(first + args.warmup + i)
    host_ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3   # time the host needs to queue a step
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3

    out = {
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "data": "synthetic",
        "host_ms_per_step": round(host_ms_per_step, 4),
    }
    if args.workload == "linear":
        value = flops_step / (ms_per_step * 1e-3) / 1e12
        launch = "eager" if step is eager_step else "hip graph replay"
        # package power while the steps run back to back as in the timed region (one more second of them)
        power = package_power(lambda i: step(first + i), seconds=1.0)
        eager = None
        if step is not eager_step:
            # the same steps launched from Python, for comparison (and the passes the GEMM timing instruments)
            for i in range(2):
                eager_step(first + i)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for i in range(args.steps):
                eager_step(first + 2 + i)
            e_host = (time.perf_counter() - t1) / args.steps * 1e3
            torch.cuda.synchronize()
            e_ms = (time.perf_counter() - t1) / args.steps * 1e3
            eager = {"ms_per_step": round(e_ms, 4), "host_ms_per_step": round(e_host, 4),
                     "value": round(flops_step / (e_ms * 1e-3) / 1e12, 2)}
        gf, gms, per_call = gemm_in_step_timing(eager_step, first + args.warmup + args.steps, args.steps)
        achieved = gf / (gms * 1e-3) / 1e12
        acts = "e4m3 activations out of the GEMM epilogue" if args.fp8_activations else "bf16 activations"
        out.update({
            "metric": "FP8Linear fwd+bwd TFLOP/s", "value": round(value, 2), "unit": "TFLOP/s", "dtype": "fp8",
            "config": {"workload": f"llama3-8b decoder-block linears fwd+bwd, 4096 tokens, {acts}, bf16 master weights, "
                                   "delayed scaling hist 16, fresh seeded X/dY and perturbed weights every step",
                       "weight_requantisation": "second stream, per layer" if args.weight_stream else "compute stream, one batched call per step",
                       "launch": launch, "launch_note": graph_note, "eager_launches": eager,
                       "package_power_during_steps": power,
                       "tokens": TOKENS, "linears": [f"{n}:{k}->{o}" for n, k, o in LINEARS], "input_sets": len(sets),
                       "flags": flags_of(args), "flops_per_step": flops_step, "pct_fp8_peak": round(100 * value / PEAK_FP8_TFLOPS, 2)},
            "verified": ({"against": "CPU oracle, steps 0 and 1: amax / scales / histories / fp8 bytes bit-exact, "
                                     "Y / dX / dW on sampled rows", "worst_rel_l2": verified} if verified is not None else False),
            "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(achieved / PEAK_FP8_TFLOPS, 4),
                         "traffic": traffic["gemm"],
                         "traffic_unit": "bytes per step over all GEMM launches: fills of the eight XCD L2s (FETCH_SIZE) + writes "
                                         "(WRITE_SIZE); L2-fill traffic, not HBM bytes (re-fetched panels can come from the "
                                         "256 MB memory-side cache)",
                         "traffic_source": traffic["source"],
                         "algorithmic_bytes": gemm_algorithmic_bytes(),
                         "kernel": "gemm_nt_big_kernel", "timing": "HIP events around every GEMM call inside the step",
                         "gemm_ms_per_step": round(gms, 4), "calls": per_call},
        })
        if args.kernel_reps > 0:
            out["roofline"]["isolated"] = gemm_isolated_timing(mods, sets, args.kernel_reps)
        del mods, sets
        torch.cuda.empty_cache()
        # secondary figure of the metric: the fused quantise kernel on configuration 2
        out["quant"] = quant_report(device, traffic)
        if not args.no_cpu_baseline:
            out["cpu_baseline"] = cpu_baseline_linear()
    else:
        value = bytes_step / (ms_per_step * 1e-3) / 1e9
        qms = quant_kernel_ms(bufs, states, 64)
        qb = 3.0 * 4096 * 4096
        q_avg = sum(qms.values()) / len(qms)
        out.update({
            "metric": "amax+quant GB/s", "value": round(value, 1), "unit": "GB/s", "dtype": "bf16->fp8",
            "config": {"workload": "bf16 [4096,4096] delayed-scaling quantise, e4m3 + e5m2 per step, hist 16",
                       "bytes_per_step": bytes_step, "pct_hbm_peak": round(100 * value / PEAK_HBM_GBPS, 2)},
            "roofline": {"bound": "hbm", "achieved": round(qb / (q_avg * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBPS,
                         "unit": "GB/s", "frac": round(qb / (q_avg * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4),
                         "traffic": traffic["quant"], "traffic_source": traffic["source"], "algorithmic_bytes": qb,
                         "kernel": "quant_flat_kernel", "ms": {k: round(v, 5) for k, v in qms.items()}},
        })
        yard = stream_probe_ms(bufs, 64)
        out["roofline"]["frac_of_yardstick"] = round(yard["read_2B_write_1B"] / q_avg, 4)
        out["yardstick"] = {"what": "ntfp8_stream_probe on the same tensors: same grid and 128-bit streaming accesses, no arithmetic, "
                                    "no reduction; copy_by_torch: the same copy by torch's copy_",
                            **{k: {"ms": round(v, 5), "GBps": round(b * 4096 * 4096 / (v * 1e-3) / 1e9, 1)}
                               for (k, v), b in zip(yard.items(), (2.0, 3.0, 4.0, 4.0))}}
        if not args.no_cpu_baseline:
            out["cpu_baseline"] = cpu_baseline_quant()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
