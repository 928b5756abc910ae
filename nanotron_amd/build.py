"""Builds nanotron_amd/libntfp8.so (the C-ABI library of include/ntfp8.h) with hipcc for gfx950.

    python -m nanotron_amd.build               the product library
    python -m nanotron_amd.build --profiling   also the profiling libraries that `bench.py --workload wg-timeline` loads

The libraries are built in-tree so that they travel with the source tree to the GPU box; nothing is
JIT-compiled at import time.

Profiling libraries (nanotron_amd/profiling/, loaded by nothing but the benchmark's wg-timeline workload):
libntfp8_stamps.so is the product library with per-workgroup time stamps compiled into the GEMM kernel
(-DNTFP8_STAMPS); the libntfp8_<experiment>.so beside it carry the same stamps and one timing experiment each on the
K loop of the forward GEMM (parts of the loop left out, or idle cycles put in; their results are wrong by design).
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libntfp8.so")
PROFILING_DIR = os.path.join(HERE, "profiling")
LIB_STAMPS = os.path.join(PROFILING_DIR, "libntfp8_stamps.so")
SOURCES = ["quant.hip", "gemm.hip", "capi.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    # packed fp32 VALU ops are kept out of every kernel
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
# name -> extra defines of gemm.hip: what the K loop of a whole tile costs, piece by piece (NTFP8_KNOCKOUT bits: 1 global
# loads, 2 deposits into LDS, 4 barrier, 8 B-fragment reads, 16 A-fragment reads), and what idle cycles cost
EXPERIMENTS = {
    "base": [],
    "no_loads": ["-DNTFP8_KNOCKOUT=1"],
    "no_loads_no_deposits": ["-DNTFP8_KNOCKOUT=3"],
    "no_barrier": ["-DNTFP8_KNOCKOUT=4"],
    "no_lds_reads": ["-DNTFP8_KNOCKOUT=24"],
    "mfma_only": ["-DNTFP8_KNOCKOUT=31"],
    "idle_256": ["-DNTFP8_IDLE=4"],
    "idle_512": ["-DNTFP8_IDLE=8"],
    "mfma_only_32x32x64": ["-DNTFP8_KNOCKOUT=31", "-DNTFP8_MFMA32=1"],
    "columns_224": ["-DNTFP8_COLUMNS=7"],
    "columns_192": ["-DNTFP8_COLUMNS=6"],
}


def experiment_lib(name: str) -> str:
    return os.path.join(PROFILING_DIR, f"libntfp8_{name}.so")


def _compile(job) -> str:
    src, defines, suffix = job
    obj = os.path.join(CSRC, src.replace(".hip", suffix + ".o"))
    cmd = [HIPCC, *FLAGS, *defines, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def _link(out: str, objs) -> None:
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out, *objs])


def build(verbose: bool = True, profiling: bool = False) -> str:
    jobs = [(s, [], "") for s in SOURCES]
    if profiling:
        jobs.append(("gemm.hip", ["-DNTFP8_STAMPS"], "_stamps"))
        jobs += [("gemm.hip", ["-DNTFP8_STAMPS", "-DNTFP8_PROFILE_NARROW", *defs], "_x_" + name)
                 for name, defs in EXPERIMENTS.items()]
    with ThreadPoolExecutor(max_workers=min(len(jobs), 6)) as ex:
        objs = list(ex.map(_compile, jobs))
    plain = objs[:len(SOURCES)]
    _link(LIB, plain)
    built = [LIB]
    if profiling:
        os.makedirs(PROFILING_DIR, exist_ok=True)
        for obj, out in zip(objs[len(SOURCES):], [LIB_STAMPS] + [experiment_lib(n) for n in EXPERIMENTS]):
            _link(out, [obj if o.endswith("gemm.o") else o for o in plain])
            built.append(out)
    if verbose:
        print("built " + " ".join(os.path.relpath(b, HERE) for b in built))
    return LIB


if __name__ == "__main__":
    build(profiling="--profiling" in sys.argv[1:])
