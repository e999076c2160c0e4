"""A per-kernel profiler over the kernel library's entry points (reference: KernelProfiler,
engine/include/llm/profile.h:35-96 and engine/src/profile.cpp:17-121 -- begin/end bracket launches
with pooled events, one synchronisation when the numbers are read, per name {calls, ms, flops,
bytes}; the cost of a launch is worked out beside the call, engine/src/model.cpp:76-256).

Every call into the library goes through ``library.call``; while the profiler is enabled that
function brackets the call with two events and notes the work the caller states for it: the
floating-point operations that the result needs, the bytes that have to be read and written at
least (every operand once) and, where a kernel knowingly reads an operand more than once (every
workgroup of the weight-streaming product reads all its rows of x; every workgroup of prompt attention
walks the keys before its rows), the bytes its workgroups ask for in all -- the reference's ideal and
moved bytes (engine/include/llm/profile.h:35-43); their quotient is the re-read factor.  A captured graph replays its kernels without passing here, so a
profiled run has to launch its steps one kernel at a time (``Executor.use_graphs = False``).
"""
from __future__ import annotations

import dataclasses
from typing import Callable, Dict, List, Optional, Tuple


@dataclasses.dataclass
class KernelStat:
    name: str
    calls: int = 0
    ms: float = 0.0
    flops: float = 0.0
    bytes: float = 0.0          # what the call has to move at least
    moved: float = 0.0          # what its workgroups ask for in all (>= bytes: operands read again)


def _device_event():
    import torch
    return torch.cuda.Event(enable_timing=True)


class KernelProfiler:
    def __init__(self, new_event: Callable = _device_event):
        self.enabled = False
        self._new_event = new_event
        self._pool: List = []
        self._open: List[Tuple[str, object, object, float, float, float]] = []
        self._stats: Dict[str, KernelStat] = {}

    def enable(self, on: bool) -> None:
        self.enabled = bool(on)

    def reset(self) -> None:
        self.flush()
        self._stats.clear()

    def _event(self):
        return self._pool.pop() if self._pool else self._new_event()

    def begin(self, name: str, cost: Optional[Callable[[], Tuple[float, float]]]):
        """Marks the start of a launch; returns what end() needs."""
        work = cost() if cost is not None else (0.0, 0.0)
        flops, nbytes = work[0], work[1]
        moved = work[2] if len(work) > 2 else nbytes
        start, stop = self._event(), self._event()
        start.record()
        return (name, start, stop, float(flops), float(nbytes), float(moved))

    def end(self, token) -> None:
        token[2].record()
        self._open.append(token)

    def flush(self) -> None:
        """Waits for the launches bracketed so far and adds their times up."""
        for name, start, stop, flops, nbytes, moved in self._open:
            stop.synchronize()
            s = self._stats.setdefault(name, KernelStat(name))
            s.calls += 1
            s.ms += start.elapsed_time(stop)
            s.flops += flops
            s.bytes += nbytes
            s.moved += moved
            self._pool.extend((start, stop))
        self._open.clear()

    def stats(self) -> List[KernelStat]:
        """Per name, the slowest first."""
        self.flush()
        return sorted(self._stats.values(), key=lambda s: -s.ms)


_profiler = KernelProfiler()


def profiler() -> KernelProfiler:
    return _profiler
