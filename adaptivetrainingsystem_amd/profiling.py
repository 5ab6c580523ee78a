"""Stage timing with HIP events on the stream the kernels run on.

The reference times its MoE ops with wall-clock and two device synchronisations
per call (Src/Main_Scripts/core/moe_cuda_wrapper.py:76-159).  Here a stage is
bracketed by two events recorded on the current stream; nothing synchronises
until `summary()` is asked for.
"""
from __future__ import annotations

from collections import OrderedDict
from contextlib import contextmanager
from typing import Dict, List, Tuple

import torch


class StageTimer:
    """`only`: names of the stages to bracket (the others run untimed).  An event pair costs the stream about
    10 us, which is a tenth of a decode-sized step if every stage is bracketed."""

    def __init__(self, only=None):
        self._events: "OrderedDict[str, List[Tuple[torch.cuda.Event, torch.cuda.Event]]]" = OrderedDict()
        self._only = None if only is None else frozenset(only)

    @contextmanager
    def range(self, name: str):
        if self._only is not None and name not in self._only:
            yield
            return
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        start.record()
        try:
            yield
        finally:
            stop.record()
            self._events.setdefault(name, []).append((start, stop))

    def reset(self) -> None:
        self._events.clear()

    def summary(self) -> Dict[str, Dict[str, float]]:
        """Synchronises once and returns {stage: {calls, mean_ms, min_ms, total_ms, median_ms, max_ms}}."""
        torch.cuda.synchronize()
        out = {}
        for name, pairs in self._events.items():
            ms = [a.elapsed_time(b) for a, b in pairs]
            out[name] = {"calls": len(ms), "mean_ms": sum(ms) / len(ms), "min_ms": min(ms), "total_ms": sum(ms),
                         "median_ms": sorted(ms)[len(ms) // 2], "max_ms": max(ms)}
        return out


@contextmanager
def _null_range():
    yield


def stage(timer, name: str):
    return timer.range(name) if timer is not None else _null_range()
