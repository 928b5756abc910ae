"""Builds nanotron_amd/libntfp8.so (the C-ABI library of include/ntfp8.h) with hipcc for gfx950, and beside it
libntfp8_stamps.so, the same library with per-workgroup time stamps compiled into the GEMM kernel (-DNTFP8_STAMPS;
only `bench.py --workload wg-timeline` loads it).

    python -m nanotron_amd.build

The library is built in-tree so that it travels with the source tree to the GPU box; nothing is
JIT-compiled at import time.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libntfp8.so")
LIB_STAMPS = os.path.join(HERE, "libntfp8_stamps.so")
SOURCES = ["quant.hip", "gemm.hip", "capi.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    # packed fp32 VALU ops are kept out of every kernel
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


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


def build(verbose: bool = True) -> str:
    jobs = [(s, [], "") for s in SOURCES] + [("gemm.hip", ["-DNTFP8_STAMPS"], "_stamps")]
    with ThreadPoolExecutor(max_workers=len(jobs)) as ex:
        objs = list(ex.map(_compile, jobs))
    plain, stamped = objs[:len(SOURCES)], objs[len(SOURCES)]
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *plain])
    with_stamps = [stamped if o.endswith("gemm.o") else o for o in plain]
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_STAMPS, *with_stamps])
    if verbose:
        print(f"built {LIB} and {LIB_STAMPS}")
    return LIB


if __name__ == "__main__":
    build()
