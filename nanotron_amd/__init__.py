"""MI355X-native implementation of nanotron's FP8 linear hot path (`nanotron.fp8`).

`nanotron_amd.fp8` mirrors the reference package's public names one to one; the arithmetic is done
by hand-written gfx950 HIP kernels behind the C ABI of include/ntfp8.h (libntfp8.so).
"""
import sys

__version__ = "0.1.0"


def install_as_nanotron_fp8() -> None:
    """Register nanotron_amd.fp8 under the reference's import path, so that existing code doing
    `from nanotron.fp8 import FP8Linear` (src/nanotron/fp8/__init__.py:3-6) picks up this
    implementation without edits."""
    import importlib
    import types

    from . import fp8

    if "nanotron" not in sys.modules:
        try:
            importlib.import_module("nanotron")
        except Exception:
            pkg = types.ModuleType("nanotron")
            pkg.__path__ = []
            sys.modules["nanotron"] = pkg
    sys.modules["nanotron.fp8"] = fp8
    setattr(sys.modules["nanotron"], "fp8", fp8)
    for sub in ("constants", "dtypes", "kernel", "linear", "meta", "parameter", "tensor", "utils"):
        sys.modules[f"nanotron.fp8.{sub}"] = importlib.import_module(f"nanotron_amd.fp8.{sub}")
