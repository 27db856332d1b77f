"""`Trace` under the reference's name (RPEG/schedule/trace.py:18-118): start and finish time of every lowered node
and the allocations the scheduler reserved for it.  The times and the reservations come from the engine; the two
summary metrics fold them on the host exactly as the reference does, device by device in the insertion order of its
dictionaries, so they equal the reference's floats."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional

from ..core.types import Allocation


def _devices(alloc: Allocation):
    o, e = alloc.origin, alloc.extent
    return [(r, n, g) for r in range(o[0], o[0] + e[0]) for n in range(o[1], o[1] + e[1])
            for g in range(o[2], o[2] + e[2])]


@dataclass(frozen=True)
class Trace:
    start: Dict[object, float]
    finish: Dict[object, float]
    reserved_allocations: Optional[dict] = None

    def makespan(self) -> float:
        return max(self.finish.values())

    def throughput(self, W_step: float, K: int) -> float:
        return K * W_step / self.makespan()

    def utilization(self) -> float:
        """Mean over the devices any node reserves of merged busy time / makespan (trace.py:53-101)."""
        ms = self.makespan()
        if ms <= 0:
            return 0.0
        intervals: Dict[tuple, list] = {}
        for node, s in self.start.items():
            allocs = (self.reserved_allocations[node] if self.reserved_allocations is not None
                      else node.allocs[-1:] if node.kind in ("comm", "reshard") else node.allocs)
            for alloc in allocs:
                for dv in _devices(alloc):
                    intervals.setdefault(dv, []).append((s, self.finish[node]))
        if not intervals:
            return 0.0
        total = 0.0
        for spans in intervals.values():
            merged = 0.0
            cs = ce = None
            for s, e in sorted(spans):
                if ce is None or s > ce:
                    if ce is not None:
                        merged += ce - cs
                    cs, ce = s, e
                else:
                    ce = max(ce, e)
            if ce is not None:
                merged += ce - cs
            total += merged / ms
        return total / len(intervals)

    def n_active(self) -> int:
        """Number of devices inside any allocation of any node (trace.py:103-118)."""
        devices = set()
        for node in self.start:
            for alloc in node.allocs:
                devices.update(_devices(alloc))
        return len(devices)
