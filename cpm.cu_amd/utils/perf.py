"""Label-keyed timers, switched on at run time.

The reference compiles its timers in with -DENABLE_PERF and prints a table of
label, count, total and average (src/perf.cuh:18-289).  Here a timer is a
context manager; GPU timers bracket the work with events on the current stream
and read them when the summary is made, so that timing adds no synchronisation
to the steps themselves.
"""
from __future__ import annotations

import sys
import time
from contextlib import contextmanager
from typing import Dict, List, Tuple

import torch


class PerfTimers:
    def __init__(self, enabled: bool = False):
        self.enabled = enabled
        self._cpu: Dict[str, List[float]] = {}
        self._gpu: Dict[str, List[Tuple[torch.cuda.Event, torch.cuda.Event]]] = {}

    @contextmanager
    def cpu(self, label: str):
        if not self.enabled:
            yield
            return
        t0 = time.perf_counter()
        try:
            yield
        finally:
            self._cpu.setdefault(label, []).append((time.perf_counter() - t0) * 1e3)

    @contextmanager
    def gpu(self, label: str):
        if not self.enabled:
            yield
            return
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        try:
            yield
        finally:
            b.record()
            self._gpu.setdefault(label, []).append((a, b))

    def summary(self) -> List[Tuple[str, str, int, float, float]]:
        rows = []
        for label, ms in self._cpu.items():
            rows.append((label, "cpu", len(ms), sum(ms), sum(ms) / len(ms)))
        if self._gpu:
            torch.cuda.synchronize()
        for label, evs in self._gpu.items():
            ms = [a.elapsed_time(b) for a, b in evs]
            rows.append((label, "gpu", len(ms), sum(ms), sum(ms) / len(ms)))
        return rows

    def print_summary(self, file=None):
        file = file or sys.stdout
        rows = self.summary()
        if not rows:
            return
        print(f"{'label':<28}{'type':<6}{'count':>8}{'total ms':>12}{'avg ms':>12}", file=file)
        for label, kind, n, tot, avg in rows:
            print(f"{label:<28}{kind:<6}{n:>8}{tot:>12.3f}{avg:>12.3f}", file=file)
        if torch.cuda.is_available():
            free, total = torch.cuda.mem_get_info()
            print(f"GPU memory: {(total - free) / 2**30:.2f} GiB used of {total / 2**30:.2f} GiB", file=file)
