"""Timing helpers (reference: vectorlink_gpu/log.py).  The reference's decorator is
effectively always on because its DEBUG is None or a string, never False
(log.py:24); here it wraps only when VECTORLINK_DEBUG is set."""
import time

import torch

from .constants import DEBUG

CLOSEST_VECTORS_BATCH_TIME = 0.0


def timed(fn):
    wall_start = time.time()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    result = fn()
    end.record()
    torch.cuda.synchronize()
    wall_end = time.time()
    return result, start.elapsed_time(end) / 1_000, (wall_end - wall_start)


def log_time(func):
    if not DEBUG:
        return func

    def wrapper(*args, **kwargs):
        global CLOSEST_VECTORS_BATCH_TIME
        (result, gpu_time, wall_time) = timed(lambda: func(*args, **kwargs))
        print(f"[{func.__name__}]\n\tGPU time: {gpu_time}\n\tWALL time {wall_time}")
        if func.__name__ == "closest_vectors":
            CLOSEST_VECTORS_BATCH_TIME = max(wall_time, CLOSEST_VECTORS_BATCH_TIME)
        return result

    wrapper.__name__ = func.__name__
    return wrapper
