"""The two pieces of DualPipeV state the expert path has to honour.

Mirrors ``pithtrain/dualpipe/utils.py``: ``FP8WeightCacheControl`` (:24-53) versions the per-module
quantised-weight caches so a weight is quantised once per pipeline step, and ``WeightGradStore``
(:56-80) is the FIFO that lets the pipeline run weight-gradient closures later than the
input-gradient pass (zero-bubble W phase).
"""

from __future__ import annotations

import queue
from typing import Callable, List

import torch.nn as nn


class FP8WeightCacheControl:
    """Global version number; a module re-quantises its weight when its cached version differs."""

    version: int = 0

    @classmethod
    def step(cls) -> None:
        cls.version += 1

    @classmethod
    def clear(cls, *modules: nn.Module) -> None:
        """Drop cached FP8 weights (``_wq_cache``, and the fused gate/up operand ``_gu_cache`` of
        expert blocks with separate projections) of every submodule to free memory."""
        for root in modules:
            for m in root.modules():
                if hasattr(m, "_wq_cache"):
                    m._wq_cache = None
                if hasattr(m, "_gu_cache"):
                    m._gu_cache = None


class WeightGradStore:
    """Deferred weight-gradient closures: ``put`` while a backward runs, ``flush`` to seal the
    batch, ``pop`` to execute the oldest sealed batch."""

    enabled: bool = False
    cache: List[Callable] = []
    funcs_queue: "queue.Queue[List[Callable]]" = queue.Queue()

    @classmethod
    def put(cls, func: Callable) -> None:
        cls.cache.append(func)

    @classmethod
    def flush(cls) -> None:
        cls.funcs_queue.put(cls.cache)
        cls.cache = []

    @classmethod
    def pop(cls) -> None:
        assert not cls.funcs_queue.empty(), "Pop empty queue."
        for func in cls.funcs_queue.get():
            func()

    @classmethod
    def clear(cls) -> None:
        cls.cache = []
        cls.funcs_queue = queue.Queue()
