"""Named ranges around the phases of an engine step, for a profiler's timeline.

The reference wraps its scheduling, prefill and decode in ``record_function`` ranges
(``serving/engine.py:334,342,359``).  Here a range is both a ``torch.profiler`` range and, on the GPU
platform, a roctx range (``torch.cuda.nvtx`` is roctx there), which ``rocprofv3 --marker-trace`` shows
beside the kernels.  Switched off (the default) a range is one shared object that does nothing.
"""

from __future__ import annotations

import contextlib


class _Nothing:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NOTHING = _Nothing()


class NamedRanges:
    def __init__(self, enabled: bool = False):
        self.enabled = bool(enabled)
        self._markers = None
        self._record = None
        if self.enabled:
            import torch
            self._record = torch.profiler.record_function
            try:
                from torch.cuda import nvtx
                if torch.cuda.is_available():
                    nvtx.range_push("simple-inference_amd ranges on")
                    nvtx.range_pop()
                    self._markers = nvtx
            except Exception:    # this torch was built without marker support: the profiler ranges remain
                self._markers = None
        self.entered = []    # names in the order they were entered (tests read it)

    def __call__(self, name: str):
        return self._range(name) if self.enabled else _NOTHING

    @contextlib.contextmanager
    def _range(self, name: str):
        self.entered.append(name)
        if self._markers is not None:
            self._markers.range_push(name)
        try:
            with self._record(name):
                yield
        finally:
            if self._markers is not None:
                self._markers.range_pop()
