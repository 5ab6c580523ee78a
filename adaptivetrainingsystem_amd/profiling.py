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
        """Synchronises once and returns {stage: {calls, mean_ms, min_ms, total_ms, median_ms, p10_ms, p90_ms,
        max_ms}} (percentiles by nearest rank)."""
        torch.cuda.synchronize()
        out = {}
        for name, pairs in self._events.items():
            ms = sorted(a.elapsed_time(b) for a, b in pairs)
            n = len(ms)
            out[name] = {"calls": n, "mean_ms": sum(ms) / n, "min_ms": ms[0], "total_ms": sum(ms),
                         "median_ms": ms[n // 2], "p10_ms": ms[min(n - 1, int(0.1 * n))],
                         "p90_ms": ms[min(n - 1, int(0.9 * n))], "max_ms": ms[-1]}
        return out


class MoEPerformanceMonitor:
    """The reference's monitor of its MoE operators (Src/Main_Scripts/core/moe_cuda_wrapper.py:76-136), with the
    same fields, methods and `get_stats` keys.  The reference brackets every operator call with two device
    synchronisations; here `timer_context` records a pair of HIP events on the launch stream and the elapsed
    times are read only when the statistics are asked for.  There is no PyTorch fallback in this build, so
    the `pytorch_*` side only ever moves if a caller records into it."""

    def __init__(self):
        self.reset()

    def reset(self) -> None:
        self.cuda_time = 0.0
        self.pytorch_time = 0.0
        self.cuda_calls = 0
        self.pytorch_calls = 0
        self.cuda_tokens = 0
        self.pytorch_tokens = 0
        self._pending: List[Tuple[torch.cuda.Event, torch.cuda.Event, bool]] = []

    def record_cuda(self, time_ms: float, num_tokens: int) -> None:
        self.cuda_time += time_ms
        self.cuda_calls += 1
        self.cuda_tokens += num_tokens

    def record_pytorch(self, time_ms: float, num_tokens: int) -> None:
        self.pytorch_time += time_ms
        self.pytorch_calls += 1
        self.pytorch_tokens += num_tokens

    _PENDING_BOUND = 1024

    def _record_events(self, start, stop, use_cuda: bool, num_tokens: int) -> None:
        self._pending.append((start, stop, use_cuda))
        if len(self._pending) > self._PENDING_BOUND:
            self._collect_finished()
        if use_cuda:
            self.cuda_calls += 1
            self.cuda_tokens += num_tokens
        else:
            self.pytorch_calls += 1
            self.pytorch_tokens += num_tokens

    def _add_elapsed(self, start, stop, use_cuda: bool) -> None:
        ms = start.elapsed_time(stop)
        if use_cuda:
            self.cuda_time += ms
        else:
            self.pytorch_time += ms

    def _collect_finished(self) -> None:
        """Reads the pairs whose stop event has already completed, without synchronising, so a loop that
        monitors for a long time and seldom asks for statistics holds a bounded number of events.  If the
        device is more than a bound's worth of calls behind the host, the oldest pair is waited for."""
        keep = []
        for start, stop, use_cuda in self._pending:
            if stop.query():
                self._add_elapsed(start, stop, use_cuda)
            else:
                keep.append((start, stop, use_cuda))
        if len(keep) > self._PENDING_BOUND:
            keep[0][1].synchronize()
            self._add_elapsed(*keep[0])
            keep = keep[1:]
        self._pending = keep

    def _drain(self) -> None:
        if not self._pending:
            return
        torch.cuda.synchronize()
        for start, stop, use_cuda in self._pending:
            self._add_elapsed(start, stop, use_cuda)
        self._pending = []

    def get_stats(self) -> Dict[str, float]:
        self._drain()
        total_time = self.cuda_time + self.pytorch_time
        if total_time == 0:
            return {"status": "No data yet"}
        return {
            "cuda_calls": self.cuda_calls,
            "pytorch_calls": self.pytorch_calls,
            "cuda_time_ms": self.cuda_time,
            "pytorch_time_ms": self.pytorch_time,
            "cuda_percentage": self.cuda_time / total_time * 100,
            "estimated_speedup": (self.pytorch_time / self.cuda_time) if self.cuda_time > 0 else 1.0,
            "tokens_per_sec_cuda": (self.cuda_tokens / (self.cuda_time / 1000)) if self.cuda_time > 0 else 0,
            "tokens_per_sec_pytorch": (self.pytorch_tokens / (self.pytorch_time / 1000)) if self.pytorch_time > 0 else 0,
        }

    def print_summary(self) -> None:
        stats = self.get_stats()
        if "status" in stats:
            print(f"\n{stats['status']}")
            return
        print(f"\n{'=' * 70}\nMoE operator summary (gfx950 kernels)\n{'=' * 70}")
        print(f"Kernel calls:   {stats['cuda_calls']:,}")
        print(f"Kernel time:    {stats['cuda_time_ms']:.2f} ms")
        print(f"Throughput:     {stats['tokens_per_sec_cuda']:,.0f} tokens/sec")
        if stats["pytorch_calls"]:
            print(f"Other calls:    {stats['pytorch_calls']:,} ({stats['pytorch_time_ms']:.2f} ms)")
        print("=" * 70)


_GLOBAL_MONITOR = MoEPerformanceMonitor()
_MONITOR_ENABLED = False


def enable_performance_monitor(on: bool = True) -> None:
    """The `MoECUDAOps` operators record into the global monitor only while this is on (an event pair per call
    costs the stream about 10 us; the reference pays two synchronisations per call unconditionally)."""
    global _MONITOR_ENABLED
    _MONITOR_ENABLED = bool(on)


@contextmanager
def timer_context(use_cuda: bool, num_tokens: int):
    """moe_cuda_wrapper.py:142-159 without the synchronisations: the bracket is a pair of HIP events."""
    if not _MONITOR_ENABLED:
        yield
        return
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    try:
        yield
    finally:
        stop.record()
        _GLOBAL_MONITOR._record_events(start, stop, use_cuda, num_tokens)


def get_performance_summary():
    return _GLOBAL_MONITOR.get_stats()


def print_performance_summary() -> None:
    _GLOBAL_MONITOR.print_summary()


def reset_performance_monitor() -> None:
    _GLOBAL_MONITOR.reset()


@contextmanager
def _null_range():
    yield


def stage(timer, name: str):
    return timer.range(name) if timer is not None else _null_range()


def calibrate_mfma(shape: str = "16x16x32", random_operands: bool = True, iters: int = 0, reps: int = 4):
    """MFMA-only loop (operands in registers, no memory traffic): what the matrix cores sustain on this
    machine with all-zero or with random bf16 operands.  Returns {"tflops", "core_clock_mhz", "ms"} of the
    last of `reps` back-to-back launches (the core clock settles during the first ones)."""
    import ctypes

    from . import _lib
    from .ops import _stream
    code = {"32x32x16": 0, "16x16x32": 1}[shape]
    iters = iters or (16000 if code == 0 else 8000)     # about 4 ms per launch
    lib = _lib.load()
    clocks = torch.zeros(2, dtype=torch.int64, device="cuda")
    flop = ctypes.c_double(0.0)
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(reps):
        ev0.record()
        _lib.check(lib.ats_calibrate_mfma(code, int(random_operands), iters, clocks.data_ptr(), ctypes.byref(flop),
                                          _stream()), "ats_calibrate_mfma")
        ev1.record()
    torch.cuda.synchronize()
    ms = ev0.elapsed_time(ev1)
    c = clocks.cpu().tolist()
    return {"tflops": flop.value / (ms * 1e-3) / 1e12, "core_clock_mhz": 100.0 * c[0] / max(c[1], 1), "ms": ms}


def stream_copy(src: torch.Tensor, dst: torch.Tensor) -> None:
    """The library's plain streaming copy (16 bytes per lane, four loads in flight): the yardstick for the
    bandwidth-bound kernels."""
    from . import _lib
    from .ops import _stream
    if not (src.is_cuda and dst.is_cuda and src.is_contiguous() and dst.is_contiguous()) or \
            src.numel() * src.element_size() != dst.numel() * dst.element_size():
        raise _lib.AtsError("stream_copy: contiguous GPU tensors of the same size")
    _lib.check(_lib.load().ats_calibrate_copy(src.data_ptr(), dst.data_ptr(), src.numel() * src.element_size(),
                                              _stream()), "ats_calibrate_copy")


def stream_read(src: torch.Tensor, sink: torch.Tensor) -> None:
    """The library's plain streaming read (16 bytes per lane, eight loads in flight): the yardstick for the
    kernels that stream weights.  `sink`: any GPU tensor of at least 4 bytes (not written in practice)."""
    from . import _lib
    from .ops import _stream
    if not (src.is_cuda and sink.is_cuda and src.is_contiguous()) or sink.numel() * sink.element_size() < 4:
        raise _lib.AtsError("stream_read: a contiguous GPU tensor and a GPU sink of at least 4 bytes")
    _lib.check(_lib.load().ats_calibrate_read(src.data_ptr(), src.numel() * src.element_size(), sink.data_ptr(),
                                              _stream()), "ats_calibrate_read")
