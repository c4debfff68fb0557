"""Optional per-kernel timing of the operator.

A benchmark installs a ``KernelTimer``; the launch helpers then record an event on the
launch stream before and after every kernel (the backward is issued as its two kernels,
one C call each, via SbaParams.bwd_phases).  With no timer installed -- the normal
case -- nothing is recorded and the backward is a single C call.

Every event record is a marker packet in the GPU queue that the neighbouring kernels wait
for (several microseconds each, five per forward + backward), so a timer can sample:
``KernelTimer(every=5)`` with ``next_step()`` called once per step instruments every fifth
step and leaves the others untouched.
"""
from __future__ import annotations

import ctypes as C
from collections import defaultdict
from typing import Optional

import torch

from .. import _lib

_TIMER: Optional["KernelTimer"] = None


class KernelTimer:
    """Collects (name, start_event, end_event) triples; durations after a synchronize."""

    def __init__(self, every: int = 1):
        self._last = None
        self._spans = []
        self.every = max(1, int(every))
        self._step = -1
        self.active = True               # until next_step() is first called: every launch

    def next_step(self):
        self._step += 1
        self.active = self._step % self.every == 0

    def mark(self, name: str):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()                      # torch's current stream = the stream we launch on
        if name != "start" and self._last is not None:
            self._spans.append((name, self._last, ev))
        self._last = ev

    def durations_ms(self):
        out = defaultdict(list)
        for name, a, b in self._spans:
            out[name].append(a.elapsed_time(b))
        return dict(out)


def install(timer: Optional[KernelTimer]):
    global _TIMER
    _TIMER = timer


def _on() -> bool:
    return _TIMER is not None and _TIMER.active


def mark(name: str):
    if _on():
        _TIMER.mark(name)


def launch_bwd(lib, p):
    if not _on():
        _lib.check(lib.sba_bwd(C.byref(p)), "sba_bwd")
        if _lib.gave_up_checked():
            _lib.raise_if_gave_up(p)
        return
    mark("start")
    p.bwd_phases = 1
    _lib.check(lib.sba_bwd(C.byref(p)), "sba_bwd")
    # without the forward's tables the first call also rebuilds them: two kernels in one span, named for both
    mark("bwd_dq" if p.workspace else "bwd_carries_dq")
    p.bwd_phases = 2
    _lib.check(lib.sba_bwd(C.byref(p)), "sba_bwd")
    mark("bwd_dkv")
    p.bwd_phases = 0
    if _lib.gave_up_checked():
        _lib.raise_if_gave_up(p)
