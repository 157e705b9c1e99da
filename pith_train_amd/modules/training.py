"""The switch the expert path sits behind.

The reference binds ``training.fp8``, ``training.Linear`` and ``training.GroupedLinear`` once in
``setup_model`` (``pithtrain/modules/training.py:383-385``, state in
``pithtrain/contexts/training.py``); model code then instantiates ``training.Linear`` /
``training.GroupedLinear`` without knowing the precision.
"""

from __future__ import annotations

import torch.nn as nn

from ..operators import grouped_linear as _gl
from ..operators.linear import FP8Linear

fp8: bool = True
Linear = FP8Linear
GroupedLinear = _gl.FP8GroupedLinear


def setup(use_fp8: bool) -> None:
    """Select FP8 (gfx950 kernels) or BF16 (torch) layers for subsequently built modules."""
    global fp8, Linear, GroupedLinear
    fp8 = bool(use_fp8)
    Linear = FP8Linear if fp8 else nn.Linear
    GroupedLinear = _gl.FP8GroupedLinear if fp8 else _gl.GroupedLinear
