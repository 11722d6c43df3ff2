"""Per-kernel times of unrecorded steps, from event pairs around every kernel call.

The reference times whole stages with events around them
(src/examples/lib/inference_batch.cc:105, :126, :161, :226-231).  Here every call of a kernel
face (``ops.kernels``) inside ``with KernelTimer() as t:`` is bracketed by two events on the
current stream and recorded with its sizes; ``t.summary()`` groups the calls by kernel and sizes
and prices each group against the MI355X's memory and matrix peaks.  An event pair around nothing
is timed too and its mean taken off every call.  Recorded (graph) steps cannot be timed this way:
run the step unrecorded.  The kernels are the same; what a call reads from cache may differ."""
from __future__ import annotations

import statistics
from typing import Dict, List, Optional, Tuple

import torch

from . import kernels as K

HBM_PEAK_BYTES = 8.0e12
MATRIX_PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}


class KernelTimer:
    def __init__(self):
        self.calls: List[Tuple[str, dict, torch.cuda.Event, torch.cuda.Event]] = []
        self._overhead_us: Optional[float] = None

    # ---------------------------------------------------------------- recording
    def begin(self) -> torch.cuda.Event:
        e = torch.cuda.Event(enable_timing=True)
        e.record()
        return e

    def end(self, name: str, info: dict, begin: torch.cuda.Event) -> None:
        e = torch.cuda.Event(enable_timing=True)
        e.record()
        self.calls.append((name, info, begin, e))

    def __enter__(self) -> "KernelTimer":
        if K._timer is not None:
            raise RuntimeError("a kernel timer is already active")
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("kernel calls cannot be timed while a step is being recorded")
        pairs = []
        for _ in range(64):                       # what a pair costs with nothing between its events
            a = self.begin()
            b = torch.cuda.Event(enable_timing=True)
            b.record()
            pairs.append((a, b))
        torch.cuda.synchronize()
        self._overhead_us = statistics.median(a.elapsed_time(b) for a, b in pairs) * 1e3
        K._timer = self
        return self

    def __exit__(self, *exc) -> bool:
        K._timer = None
        return False

    # ------------------------------------------------------------------ results
    def summary(self, extra_bytes=None, extra_flops=None) -> List[dict]:
        """One entry per (kernel, sizes): calls, mean microseconds a call (event overhead taken
        off), and the fraction of the floor, which is the larger of bytes / HBM peak and flops /
        matrix peak.  ``extra_bytes(name, info)`` / ``extra_flops(name, info)`` supply what the
        sizes alone do not tell (the keys an attention call reads)."""
        torch.cuda.synchronize()
        groups: Dict[Tuple, List[float]] = {}
        infos: Dict[Tuple, dict] = {}
        for name, info, a, b in self.calls:
            key = (name,) + tuple(sorted((k, v) for k, v in info.items() if k not in ("bytes", "flops")))
            groups.setdefault(key, []).append(max(0.0, a.elapsed_time(b) * 1e3 - self._overhead_us))
            infos[key] = dict(info, name=name)
        out = []
        for key, times in groups.items():
            info = infos[key]
            name = info.pop("name")
            nbytes = info.pop("bytes", None)
            flops = info.pop("flops", None)
            if nbytes is None and extra_bytes is not None:
                nbytes = extra_bytes(name, info)
            if flops is None and extra_flops is not None:
                flops = extra_flops(name, info)
            us = statistics.mean(times)
            row = {"kernel": name, "sizes": info, "calls": len(times), "us_per_call": round(us, 2),
                   "us_total": round(sum(times), 1)}
            floor = 0.0
            if nbytes:
                row["GB/s"] = round(nbytes / us / 1e3, 1) if us > 0 else None
                floor = max(floor, nbytes / HBM_PEAK_BYTES * 1e6)
            if flops:
                peak = MATRIX_PEAK_FLOPS.get(info.get("dtype", "bfloat16"), MATRIX_PEAK_FLOPS["bfloat16"])
                row["TFLOP/s"] = round(flops / us / 1e6, 1) if us > 0 else None
                floor = max(floor, flops / peak * 1e6)
            if floor > 0 and us > 0:
                row["bound"] = "hbm" if nbytes and nbytes / HBM_PEAK_BYTES * 1e6 >= floor else "matrix"
                row["frac"] = round(floor / us, 4)
            out.append(row)
        out.sort(key=lambda r: -r["us_total"])
        return out
