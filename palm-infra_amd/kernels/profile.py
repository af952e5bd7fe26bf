"""Per-kernel timing of steps: the command line's ``--profile`` and ``--trace``.

The reference's engine counts calls and time per operator of its graph and prints them as
``[prefill_profile]`` and ``[decode_profile]`` tables (examples/bench.cpp:52-99), and writes a Chrome
trace if a path is given (examples/cli_common.cpp:172-176, engine/model_loader.cpp:1012).  Here every
kernel launch passes through ``library.call`` (and the library matrix product through
``ops.linear_library``), so a recorder installed there brackets each launch with two events on the
launching stream.  While a recorder is installed the engine records no HIP graphs and replays none: a
replay is one launch whose kernels cannot be told apart from the host.
"""
from __future__ import annotations

import json
from contextlib import contextmanager

_active = None


def active():
    return _active


def _events():
    import torch
    return torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)


def _synchronize():
    import torch
    torch.cuda.synchronize()


class KernelProfile:
    """Collects (section, entry point, start event, end event) of every launch while installed."""

    def __init__(self):
        self.launches: list = []      # (section, name, ev0, ev1)
        self.steps: list = []         # (section, label, ev0, ev1)
        self.section = "other"
        self._origin = None

    # ---- recording ---------------------------------------------------------------------------
    def install(self) -> "KernelProfile":
        global _active
        if _active is not None and _active is not self:
            raise RuntimeError("another kernel profile is being recorded")
        _active = self
        if self._origin is None:
            self._origin, _ = _events()
            self._origin.record()
        return self

    def remove(self) -> None:
        global _active
        if _active is self:
            _active = None

    def __enter__(self):
        return self.install()

    def __exit__(self, *exc):
        self.remove()

    def around(self, name: str, launch):
        """Run ``launch()`` between two events."""
        ev0, ev1 = _events()
        ev0.record()
        try:
            return launch()
        finally:
            ev1.record()
            self.launches.append((self.section, name, ev0, ev1))

    @contextmanager
    def step(self, section: str, label: str):
        """A step of the engine: its launches, and those that follow until the next step (the choice of
        the next token), are filed under ``section`` ("prefill" or "decode")."""
        self.section = section
        ev0, ev1 = _events()
        ev0.record()
        try:
            yield
        finally:
            ev1.record()
            self.steps.append((section, label, ev0, ev1))

    def reset(self) -> None:
        self.launches.clear()
        self.steps.clear()

    # ---- reading -----------------------------------------------------------------------------
    def rows(self, section: str) -> list:
        """[(entry point, calls, total ms)] of a section, the longest first."""
        _synchronize()
        total: dict = {}
        for sec, name, ev0, ev1 in self.launches:
            if sec != section:
                continue
            calls, ms = total.get(name, (0, 0.0))
            total[name] = (calls + 1, ms + ev0.elapsed_time(ev1))
        return sorted(((n, c, ms) for n, (c, ms) in total.items()), key=lambda r: -r[2])

    def sections(self) -> list:
        seen = []
        for sec, *_ in self.launches:
            if sec not in seen:
                seen.append(sec)
        return seen

    def format(self) -> str:
        """Tables in the reference's layout: op, calls, total_ms, avg_ms, pct (examples/bench.cpp:76-99)."""
        out = []
        for section in self.sections():
            rows = self.rows(section)
            if not rows:
                continue
            whole = sum(r[2] for r in rows)
            out.append(f"\n[{section}_profile]")
            out.append(f"  {'op':<28s} {'calls':>8s} {'total_ms':>10s} {'avg_ms':>10s} {'pct':>7s}")
            out.append(f"  {'---':<28s} {'---':>8s} {'---':>10s} {'---':>10s} {'---':>7s}")
            for name, calls, ms in rows:
                pct = 100.0 * ms / whole if whole > 0 else 0.0
                out.append(f"  {name:<28s} {calls:>8d} {ms:>10.2f} {ms / calls:>10.3f} {pct:>6.1f}%")
        return "\n".join(out)

    def chrome_trace(self) -> dict:
        """Events in the Chrome trace format (microseconds): steps on one row, launches on another."""
        _synchronize()
        events = []

        def complete(name, cat, tid, ev0, ev1):
            events.append({"name": name, "cat": cat, "ph": "X", "pid": 0, "tid": tid,
                           "ts": round(self._origin.elapsed_time(ev0) * 1000.0, 3),
                           "dur": round(ev0.elapsed_time(ev1) * 1000.0, 3)})

        for section, label, ev0, ev1 in self.steps:
            complete(label, section, 0, ev0, ev1)
        for section, name, ev0, ev1 in self.launches:
            complete(name, section, 1, ev0, ev1)
        names = [{"name": "thread_name", "ph": "M", "pid": 0, "tid": 0, "args": {"name": "steps"}},
                 {"name": "thread_name", "ph": "M", "pid": 0, "tid": 1, "args": {"name": "kernels"}}]
        return {"traceEvents": names + events, "displayTimeUnit": "ms"}

    def write_chrome_trace(self, path) -> None:
        with open(path, "w") as f:
            json.dump(self.chrome_trace(), f)
