"""Per-class kernel timing from event pairs.

The reference buckets a forward pass into embed / qkv / rope + qk-norm / kv + attention / o-proj /
ffn / final with stopwatches under ``SHARPI_CUDA_PROFILE=1``
(reference: src/SharpInference.Engine/CudaForwardPass.cs:1523-1539) and keeps a GB/s figure beside
its matvec micro-benchmark (1456-1520).  Here the parts mark what they launch with
``section(name, nbytes, flops)``; while a :class:`Profiler` is active every section is bracketed
by a pair of device events, and the report gives calls, milliseconds, bytes, GB/s and TFLOP/s per
class.  When no profiler is active a section costs one ``if``.

Event pairs measure the stream between the two records.  If the device is idle while the host is
still enqueueing, the host's latency lands inside the spans of short kernels; ``Profiler.run``
therefore keeps the device busy with filler work first, so that the whole step is already queued
when the device reaches it.
"""
from __future__ import annotations

from contextlib import contextmanager
from typing import Callable, Dict, List, Optional

import torch

_active: Optional["Profiler"] = None


class Profiler:
    def __init__(self):
        self.spans: List[tuple] = []          # (class, start event, end event, bytes, flops)
        self.depth = 0

    # -- collecting -----------------------------------------------------------
    def __enter__(self):
        global _active
        if _active is not None:
            raise RuntimeError("a profiler is already active")
        _active = self
        return self

    def __exit__(self, *exc):
        global _active
        _active = None
        return False

    def run(self, fn: Callable, filler_ms: float = 0.0, device=None):
        """fn() with this profiler active, behind `filler_ms` of filler work on the device."""
        if filler_ms > 0:
            _fill(filler_ms, device)
        with self:
            out = fn()
        torch.cuda.synchronize(device)
        return out

    # -- reporting ------------------------------------------------------------
    def table(self) -> Dict[str, dict]:
        """{class: {calls, ms, bytes, flops}} in the order the classes were first seen."""
        torch.cuda.synchronize()
        out: Dict[str, dict] = {}
        for name, a, b, nbytes, flops in self.spans:
            row = out.setdefault(name, {"calls": 0, "ms": 0.0, "bytes": 0, "flops": 0.0})
            row["calls"] += 1
            row["ms"] += a.elapsed_time(b)
            row["bytes"] += int(nbytes)
            row["flops"] += float(flops)
        return out


def format_table(table: Dict[str, dict], title: str = "", peak_gbs: float = 8000.0, peak_tflops: float = 2500.0) -> str:
    total = sum(r["ms"] for r in table.values()) or 1.0
    lines = [title] if title else []
    lines.append(f"{'class':<22}{'calls':>6}{'ms':>10}{'%':>7}{'GB':>9}{'GB/s':>9}{'of peak':>8}{'TFLOP/s':>9}{'of peak':>8}")
    for name, r in table.items():
        gbs = r["bytes"] / r["ms"] / 1e6 if r["ms"] > 0 else 0.0
        tf = r["flops"] / r["ms"] / 1e9 if r["ms"] > 0 else 0.0
        lines.append(f"{name:<22}{r['calls']:>6}{r['ms']:>10.3f}{100 * r['ms'] / total:>7.1f}{r['bytes'] / 1e9:>9.3f}"
                     f"{gbs:>9.0f}{gbs / peak_gbs:>8.2f}{tf:>9.1f}{tf / peak_tflops:>8.3f}")
    lines.append(f"{'sum':<22}{sum(r['calls'] for r in table.values()):>6}{total:>10.3f}")
    return "\n".join(lines)


def active() -> bool:
    return _active is not None


@contextmanager
def section(name: str, nbytes=0, flops=0):
    """Mark what is launched inside as one span of class `name`.  nbytes / flops: what the span
    has to move and compute (numbers, or callables asked only while profiling)."""
    p = _active
    if p is None or p.depth > 0:          # spans do not nest: the outermost counts
        if p is not None:
            p.depth += 1
        try:
            yield
        finally:
            if p is not None:
                p.depth -= 1
        return
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    p.depth += 1
    a.record()
    try:
        yield
    finally:
        b.record()
        p.depth -= 1
        p.spans.append((name, a, b, nbytes() if callable(nbytes) else nbytes, flops() if callable(flops) else flops))


_filler: dict = {}


def _fill(ms: float, device=None) -> None:
    """Queue about `ms` milliseconds of device work (large copies) without waiting for it."""
    dev = torch.device(device or "cuda")
    buf = _filler.get(dev)
    if buf is None:
        buf = _filler[dev] = (torch.empty(1 << 28, dtype=torch.uint8, device=dev), torch.empty(1 << 28, dtype=torch.uint8, device=dev))
    # 256 MiB read + 256 MiB written per copy: roughly 0.15 ms on an MI355X
    for _ in range(max(1, int(ms / 0.15))):
        buf[1].copy_(buf[0])
