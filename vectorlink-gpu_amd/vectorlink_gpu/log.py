"""Optional call timing.  Stands in for the reference's vectorlink_gpu/log.py, whose
decorator is effectively always on (its DEBUG is None or a string, never False,
log.py:24) and synchronises the device twice per call; here nothing is wrapped
unless VECTORLINK_DEBUG is set, and one synchronisation closes the measurement."""
import functools
import time

import torch

from .constants import DEBUG

# longest closest_vectors call seen so far, in wall seconds (read by ANN.dump_logs)
CLOSEST_VECTORS_BATCH_TIME = 0.0
# beam-search iterations run by closest_vectors since the import (one kernel launch each in the default form);
# a profiler's list of launches can be cut into phases with it
BEAM_ITERATIONS = 0


class _Stopwatch:
    """Wall clock plus a pair of device events around a block of work."""

    def __enter__(self):
        self.gpu = torch.cuda.is_available()
        if self.gpu:
            self._begin = torch.cuda.Event(enable_timing=True)
            self._end = torch.cuda.Event(enable_timing=True)
            self._begin.record()
        self._t0 = time.perf_counter()
        return self

    def __exit__(self, *exc):
        if self.gpu:
            self._end.record()
            torch.cuda.synchronize()
            self.device_seconds = self._begin.elapsed_time(self._end) / 1e3
        else:
            self.device_seconds = float("nan")
        self.wall_seconds = time.perf_counter() - self._t0
        return False


def timed(fn):
    """(result, device seconds, wall seconds) of calling fn()"""
    with _Stopwatch() as sw:
        result = fn()
    return result, sw.device_seconds, sw.wall_seconds


def log_time(func):
    """Decorator: print how long each call took.  A no-op unless VECTORLINK_DEBUG is set."""
    if not DEBUG:
        return func

    @functools.wraps(func)
    def timed_call(*args, **kwargs):
        global CLOSEST_VECTORS_BATCH_TIME
        with _Stopwatch() as sw:
            result = func(*args, **kwargs)
        print(f"[{func.__name__}] device {sw.device_seconds:.6f} s, wall {sw.wall_seconds:.6f} s")
        if func.__name__ == "closest_vectors" and sw.wall_seconds > CLOSEST_VECTORS_BATCH_TIME:
            CLOSEST_VECTORS_BATCH_TIME = sw.wall_seconds
        return result

    return timed_call
