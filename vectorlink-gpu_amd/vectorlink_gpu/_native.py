"""ctypes binding of libvlgpu.so (the hand-written HIP library for gfx950).

The product path never falls back to anything else: if the library is missing
or a call fails, an exception is raised.
"""
import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libvlgpu.so")
_lib = None

_i64 = C.c_int64
_ptr = C.c_void_p


class BeamParams(C.Structure):
    _fields_ = [(n, C.c_int64) for n in (
        "n_rows", "dim", "n_vectors", "width", "queue_capacity", "queue_length", "beam_size",
        "parallel_visit_count", "visit_queue_factor", "exclude_factor", "speculative_readahead", "excl_cols",
        "flags", "metric")]


METRICS = {"cosine": 0, "l2": 1}  # include/vlgpu.h: VL_METRIC_COSINE, VL_METRIC_L2


def metric_code(name: str) -> int:
    if name not in METRICS:
        raise ValueError(f"unknown metric {name!r}: expected one of {sorted(METRICS)}")
    return METRICS[name]


_SIGNATURES = {
    "vl_last_error": (C.c_char_p, []),
    "vl_version": (C.c_int, []),
    "vl_gather_distances": (C.c_int, [_ptr, _i64, _ptr, _i64, _i64, _ptr, _i64, _ptr, _ptr]),
    "vl_gather_distances_metric": (C.c_int, [_ptr, _i64, _ptr, _i64, _i64, _ptr, _i64, C.c_int, _ptr, _ptr]),
    "vl_search_from_seeds": (C.c_int, [_ptr, _i64, _i64, _ptr, _i64, _ptr, _i64, _i64, _ptr, _i64, _ptr, _ptr, _ptr]),
    "vl_search_from_seeds_metric": (C.c_int, [_ptr, _i64, _i64, _ptr, _i64, _ptr, _i64, _i64, _ptr, _i64, C.c_int, _ptr,
                                              _ptr, _ptr]),
    "vl_circulants": (C.c_int, [_ptr, _i64, _i64, _i64, _ptr, _i64, _ptr]),
    "vl_dedup_ids": (C.c_int, [_ptr, _i64, _i64, _ptr]),
    "vl_dedup_pairs": (C.c_int, [_ptr, _ptr, _i64, _i64, _ptr]),
    "vl_punchout_excluded": (C.c_int, [_ptr, _ptr, _i64, _i64, _i64, _i64, _ptr, _i64, _i64, _ptr]),
    "vl_index_by_tensor": (C.c_int, [_ptr, _ptr, _ptr, _i64, _i64, _ptr]),
    "vl_index_sort": (C.c_int, [_ptr, _ptr, _i64, _i64, _ptr]),
    "vl_punchout_duplicates": (C.c_int, [_ptr, _ptr, _i64, _i64, _ptr]),
    "vl_queue_sort": (C.c_int, [_ptr, _ptr, _i64, _i64, _ptr]),
    "vl_queue_insert": (C.c_int, [_ptr, _ptr, _i64, _i64, _i64, _ptr, _ptr, _i64, _ptr, _i64, _ptr, _ptr]),
    "vl_queue_pop": (C.c_int, [_ptr, _ptr, _i64, _i64, _i64, _ptr, _ptr]),
    "vl_seen_add": (C.c_int, [_ptr, _i64, _i64, _ptr, _i64, _ptr, C.POINTER(C.c_int), _ptr]),
    "vl_beam_workspace_bytes": (C.c_int64, [C.POINTER(BeamParams)]),
    "vl_closest_vectors": (C.c_int64, [C.POINTER(BeamParams), _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _ptr]),
    "vl_closest_vectors_noalloc": (C.c_int, [C.POINTER(BeamParams), _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _ptr, _ptr]),
    "vl_closest_vectors_with_sketch": (C.c_int64, [C.POINTER(BeamParams), _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr,
                                                   _i64, _ptr]),
    "vl_sketch_row_bytes": (C.c_int64, [_i64]),
    "vl_sketch_build": (C.c_int, [_ptr, _i64, _i64, _ptr, _ptr]),
    "vl_sketch_bounds_workspace_bytes": (C.c_int64, [_i64, _i64]),
    "vl_sketch_bounds": (C.c_int, [_ptr, _i64, _i64, _ptr, _i64, _ptr, _i64, _ptr, _ptr, _ptr, _i64, _ptr]),
    "vl_beam_profile": (C.c_int, [C.c_int, C.c_int, C.POINTER(C.c_double)]),
    "vl_beam_launches": (C.c_int64, []),
    "vl_optimize_graph_workspace_bytes": (C.c_int64, [_i64, _i64, _i64]),
    "vl_optimize_graph": (C.c_int, [_ptr, _i64, _i64, _i64, _ptr, _ptr, _i64, _ptr]),
    "vl_knn_workspace_bytes": (C.c_int64, [_i64, _i64, _i64, _i64]),
    "vl_knn_exact": (C.c_int, [_ptr, _i64, _ptr, _i64, _i64, _i64, _ptr, _ptr, _ptr, _i64, _ptr]),
    "vl_knn_exact_metric": (C.c_int, [_ptr, _i64, _ptr, _i64, _i64, _i64, C.c_int32, _ptr, _ptr, _ptr, _i64, _ptr]),
    "vl_prune": (C.c_int, [_ptr, _ptr, _i64, _i64, _ptr, _ptr, _ptr]),
}


def lib():
    """Load the library once.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python vectorlink-gpu_amd/build.py` "
                "(hipcc --offload-arch=gfx950); there is no fallback path")
        l = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def check(rc: int) -> int:
    """Turn a negative return code into an exception carrying vl_last_error()."""
    if rc < 0:
        msg = lib().vl_last_error().decode()
        if rc == -1:
            raise ValueError(msg)
        raise RuntimeError(msg)
    return rc


def ptr(t) -> C.c_void_p:
    return C.c_void_p(0 if t is None else t.data_ptr())


def stream() -> C.c_void_p:
    """The current torch stream as a hipStream_t (kernels.py:14-16 does the same for Numba)."""
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("vectorlink_gpu kernels need tensors on the GPU (there is no CPU path)")
