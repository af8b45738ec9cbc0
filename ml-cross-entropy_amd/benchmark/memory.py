"""Run time and allocator peak of one call (ref: benchmark/memory.py:13-119).

One untimed call measures memory -- the rise of the allocator's peak over the call (forward, or
backward alone when only the backward is asked for) -- then ``n_iteration`` calls are timed between
device events: from before the forward, or from after it when only the backward is timed.
"""

import gc
from dataclasses import dataclass
from typing import Callable, Optional

import torch

_PEAK = "allocated_bytes.all.peak"


class _PeakRise:
    """Bytes by which the allocator's peak rose since the last ``restart``."""

    def restart(self) -> None:
        torch.cuda.reset_peak_memory_stats()
        self._before = torch.cuda.memory_stats()[_PEAK]

    def read(self) -> int:
        torch.cuda.synchronize()
        return torch.cuda.memory_stats()[_PEAK] - self._before


def _backprop(out: torch.Tensor) -> None:
    (out if out.numel() == 1 else out.mean()).backward()


@dataclass(frozen=True)
class Stats:
    runtime_ms: float
    op_mem_mb: float

    @classmethod
    def measure(
        cls,
        f: Callable[..., torch.Tensor],
        *args,
        n_iteration: int = 1,
        forward: bool = True,
        backward: bool = False,
        pre_fn: Optional[Callable[..., None]] = None,
        **kwds,
    ) -> "Stats":
        def prepare():
            if pre_fn is not None:
                pre_fn(*args, **kwds)

        # memory: one call on a quiet allocator
        prepare()
        torch.cuda.synchronize()
        gc.collect()
        torch.cuda.empty_cache()
        rise = _PeakRise()
        rise.restart()
        out = f(*args, **kwds)
        mem_bytes = rise.read()
        if backward:
            if not forward:
                rise.restart()
            _backprop(out)
            mem_bytes = rise.read()

        # time: device events around the part that was asked for
        stream = torch.cuda.current_stream()
        spans = []
        for _ in range(n_iteration):
            prepare()
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            if forward:
                begin.record(stream)
            out = f(*args, **kwds)
            if not forward:
                begin.record(stream)
            if backward:
                _backprop(out)
            end.record(stream)
            spans.append((begin, end))
        torch.cuda.synchronize()
        total_ms = sum(b.elapsed_time(e) for b, e in spans)
        return cls(total_ms / max(n_iteration, 1), mem_bytes / 2**20)
