"""Per-kernel timing with stream events, through the library's launch hook.

``KernelTimer`` brackets every kernel the C ABI launches on the calling thread
with a pair of events recorded on the launch stream, so durations are those of
the individual kernels, measured in the same run and on the same stream as the
work being timed.
"""

from __future__ import annotations

import collections
import ctypes

import torch

from . import _lib


class KernelTimer:
    """Context manager: collects (kernel name -> list of durations in ms)."""

    def __init__(self, only=None):
        """`only`: names of the kernels to time (default: every launch). Two events on the stream per
        timed launch are not free on the device (2.5 % of a 1.1 ms step of five launches), so a
        region whose total time matters times only the kernel it needs."""

        self._only = None if only is None else frozenset(only)
        self._first = 0
        self._pending = []
        self._open = {}
        self._callback = _lib.LAUNCH_HOOK(self._on_launch)

    def _on_launch(self, _user, kernel, phase, stream):
        name = kernel.decode()
        if self._only is not None and name not in self._only:
            return
        event = torch.cuda.Event(enable_timing=True)
        event.record(torch.cuda.ExternalStream(stream) if stream else torch.cuda.current_stream())
        if phase == 0:
            self._open[name] = event
        else:
            self._pending.append((name, self._open.pop(name), event))

    def __enter__(self):
        _lib.load().ct_set_launch_hook(self._callback, None)
        return self

    def __exit__(self, *exc):
        _lib.load().ct_set_launch_hook(ctypes.cast(None, _lib.LAUNCH_HOOK), None)
        return False

    def mark(self) -> None:
        """Launches recorded up to here are left out of durations_ms (warm-up). Costs nothing on
        the device: their events are kept until the timer is read."""

        self._first = len(self._pending)

    def durations_ms(self) -> dict[str, list[float]]:
        """Synchronises and returns every launch recorded since the last mark, grouped by kernel name."""

        torch.cuda.synchronize()
        result = collections.defaultdict(list)
        for name, begin, end in self._pending[self._first:]:
            result[name].append(begin.elapsed_time(end))
        # the events are released here, in the caller's time, not whenever a later garbage
        # collection finds this object (it holds a callback that refers back to it)
        self._pending = []
        self._first = 0
        return dict(result)
