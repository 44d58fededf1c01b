"""Per-entry-point device timing with HIP events on the launch stream.

``with KernelTimer() as kt:`` brackets every C-ABI call made inside the block with a pair of
events recorded on torch's current stream (the stream the kernels are enqueued on), so the
time of each entry point can be read without a profiler.  ``kt.summary()`` synchronises once
and returns ``{entry point: {"calls": n, "total_ms": t, "avg_us": a}}``.
"""

from __future__ import annotations

from collections import defaultdict

import torch

from steptronoss_amd import _lib


class KernelTimer:
    def __init__(self):
        self._pairs = defaultdict(list)

    def __enter__(self):
        _lib.set_call_hook(self)
        return self

    def __exit__(self, *exc):
        _lib.set_call_hook(None)
        return False

    def before(self, name):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        return ev

    def after(self, name, start):
        end = torch.cuda.Event(enable_timing=True)
        end.record()
        self._pairs[name].append((start, end))

    def summary(self):
        torch.cuda.synchronize()
        out = {}
        for name, pairs in self._pairs.items():
            total = sum(a.elapsed_time(b) for a, b in pairs)
            out[name] = {"calls": len(pairs), "total_ms": total, "avg_us": 1e3 * total / max(len(pairs), 1)}
        return out

    def per_call_us(self, name):
        torch.cuda.synchronize()
        return [1e3 * a.elapsed_time(b) for a, b in self._pairs.get(name, [])]
