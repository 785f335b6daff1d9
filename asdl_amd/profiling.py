"""Profiling hooks of the path: named ranges for a tracing profiler and phase marks for a per-phase breakdown.

Ranges carry the names the reference gives its NVTX ranges -- ``cov_kron_A`` / ``cov_kron_B`` / ``cov_unit_wise``
(asdl/operations/operation.py:750, 765, 784), ``inv_kron_A_B`` (asdl/precondition/natural_gradient.py:446-451; one
range for the batched inverse of all modules instead of one per module) -- and the phase keywords of its profiling
example (examples/prof/README.md:24): ``fwd``, ``bwd``, ``upd_curv``, ``upd_inv``, ``precond``.  On ROCm
``torch.cuda.nvtx`` emits roctx ranges, which ``rocprofv3 --marker-trace`` records.

Both are off by default (a range costs about a microsecond of host time, a mark one event record):
``enable_ranges(True)`` switches the ranges on; ``set_phase_sink(list)`` makes every ``phase_mark(name)`` record a
timing event on the current stream and append ``(name, event)`` to the list, so that the caller can read the time
between consecutive marks once the device is idle."""
from contextlib import contextmanager

import time

import torch

_ranges_on = False
_phase_sink = None

__all__ = ['enable_ranges', 'ranges_enabled', 'nvtx_range', 'set_phase_sink', 'phase_mark']


def enable_ranges(flag=True):
    global _ranges_on
    _ranges_on = bool(flag) and torch.cuda.is_available()


def ranges_enabled():
    return _ranges_on


class nvtx_range:
    """asdl/utils.py:190-192.  A plain class: entered twice per hooked module and step, and a generator-based
    context manager costs a few microseconds of host time each time even when the ranges are off."""
    __slots__ = ('msg', 'on')

    def __init__(self, msg):
        self.msg = msg

    def __enter__(self):
        self.on = _ranges_on
        if self.on:
            torch.cuda.nvtx.range_push(self.msg)
        return self

    def __exit__(self, *exc):
        if self.on:
            torch.cuda.nvtx.range_pop()
        return False


def set_phase_sink(sink):
    global _phase_sink
    _phase_sink = sink


def phase_mark(name):
    """End of the phase ``name`` on the current stream (everything enqueued on it since the previous mark)."""
    if _phase_sink is None:
        return
    event = torch.cuda.Event(enable_timing=True)
    event.record()
    _phase_sink.append((name, event, time.perf_counter()))      # the host's clock too: which side bounds the phase?
