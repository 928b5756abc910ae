"""Drop-in for `nanotron.fp8` (reference: src/nanotron/fp8/__init__.py:3-6)."""
from nanotron_amd.fp8.dtypes import DTypes  # noqa
from nanotron_amd.fp8.linear import FP8Linear  # noqa
from nanotron_amd.fp8.parameter import FP8Parameter  # noqa
from nanotron_amd.fp8.tensor import DelayedScaling, FP8Tensor  # noqa
