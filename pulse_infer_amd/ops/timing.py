"""Per-entry-point timing of this package's kernels with GPU events.

``with timing.record() as table:`` brackets every call of a HIP entry point (and every
region that library products mark with ``timing.region``) with a pair of events on the
current stream; ``table.format()`` then lists calls, total and mean time per name.  It
is meant for eager steps: an event pair costs a few microseconds of its own and cannot
be recorded into a graph, so the figures say where a step's GPU time goes, not how long
a replayed step takes.
"""
from __future__ import annotations

from contextlib import contextmanager
from typing import Dict, List, Optional, Tuple

import torch

_active: Optional["Table"] = None


class Table:
    def __init__(self) -> None:
        self.pairs: List[Tuple[str, torch.cuda.Event, torch.cuda.Event]] = []

    def totals(self) -> Dict[str, Tuple[int, float]]:
        """name -> (calls, milliseconds)"""
        torch.cuda.synchronize()
        out: Dict[str, Tuple[int, float]] = {}
        for name, first, last in self.pairs:
            calls, ms = out.get(name, (0, 0.0))
            out[name] = (calls + 1, ms + first.elapsed_time(last))
        return out

    def format(self, per: int = 1) -> str:
        """A table, most expensive first; ``per`` divides calls and times (steps that were recorded)."""
        rows = sorted(self.totals().items(), key=lambda kv: -kv[1][1])
        total = sum(ms for _, (_, ms) in rows) or 1.0
        lines = [f"{'entry point':<34}{'calls':>8}{'us':>11}{'us/call':>10}{'share':>8}"]
        for name, (calls, ms) in rows:
            lines.append(f"{name:<34}{calls / per:>8.1f}{ms * 1e3 / per:>11.1f}{ms * 1e3 / calls:>10.2f}"
                         f"{100.0 * ms / total:>7.1f}%")
        lines.append(f"{'sum':<34}{sum(c for _, (c, _) in rows) / per:>8.1f}{total * 1e3 / per:>11.1f}")
        return "\n".join(lines)


def active() -> bool:
    return _active is not None


@contextmanager
def region(name: str):
    """Time what runs inside under ``name`` while a table is recording; nothing otherwise."""
    table = _active
    if table is None:
        yield
        return
    first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    first.record()
    try:
        yield
    finally:
        last.record()
        table.pairs.append((name, first, last))


@contextmanager
def record():
    global _active
    table = Table()
    previous, _active = _active, table
    try:
        yield table
    finally:
        _active = previous
