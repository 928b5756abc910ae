"""bench.py from the command line: the refusals that need no GPU, and on the GPU the switches that change which kernels
a step launches (each must still produce one JSON line with the contract's fields)."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench(*flags, timeout=280):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *flags], capture_output=True, text=True,
                          timeout=timeout, cwd=ROOT)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _bench("--gpus", "2")
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


@pytest.mark.gpu
@pytest.mark.parametrize("flags", [("--fp8-activations",), ("--transposed-copies", "--grad-transposed-copy"), ("--no-graph",)])
def test_step_variants_print_one_contract_line(flags):
    r = _bench(*flags, "--steps", "2", "--warmup", "1", "--no-cpu-baseline")
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 2 and d["value"] > 0 and d["vs_baseline"] is None
    assert d["roofline"]["bound"] == "mfma" and 0 < d["roofline"]["frac"] < 1
    assert d["config"]["launch"] == ("eager" if "--no-graph" in flags else "hip graph replay"), d["config"]["launch_note"]
    if "--fp8-activations" not in flags:
        assert d["verified"] and max(d["verified"]["worst_rel_l2"].values()) <= 1e-3
