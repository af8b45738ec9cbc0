"""Run time and allocator peak of one call (ref: benchmark/memory.py:13-119).

One untimed call measures memory -- the rise of the allocator's peak over the call (forward, or
backward alone when only the backward is asked for) -- then ``n_iteration`` calls are timed between
device events: from before the forward, or from after it when only the backward is timed.
"""

import gc
from dataclasses import dataclass
from typing import Callable, Optional

import torch


def mem_delta(s1, s0) -> int:
    return s1["allocated_bytes.all.peak"] - s0["allocated_bytes.all.peak"]


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
        if pre_fn is not None:
            pre_fn(*args, **kwds)
        torch.cuda.synchronize()
        gc.collect()
        torch.cuda.empty_cache()

        torch.cuda.reset_peak_memory_stats()
        s0 = torch.cuda.memory_stats()
        t = f(*args, **kwds)
        torch.cuda.synchronize()
        s1 = torch.cuda.memory_stats()
        if backward and not forward:
            torch.cuda.reset_peak_memory_stats()
            s0 = torch.cuda.memory_stats()
        if backward:
            if t.numel() > 1:
                t = t.mean()
            t.backward()
            torch.cuda.synchronize()
            s1 = torch.cuda.memory_stats()
        mem_bytes = mem_delta(s1, s0)

        events = []
        for _ in range(n_iteration):
            if pre_fn is not None:
                pre_fn(*args, **kwds)
            start = torch.cuda.Event(enable_timing=True)
            if forward:
                start.record(torch.cuda.current_stream())
            t = f(*args, **kwds)
            if not forward:
                start.record(torch.cuda.current_stream())
            if backward:
                if t.numel() > 1:
                    t = t.mean()
                t.backward()
            end = torch.cuda.Event(enable_timing=True)
            end.record(torch.cuda.current_stream())
            events.append((start, end))
        torch.cuda.synchronize()
        total = sum(a.elapsed_time(b) for a, b in events)
        return cls(total / max(n_iteration, 1), mem_bytes / 2**20)
