"""The C ABI without a GPU: the library loads, exports every function that
include/vlgpu.h declares, the Python binding table covers them all, and shape
validation rejects bad calls on the host before anything is launched."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "vlgpu.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vl_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from vectorlink_gpu import _native

    if not os.path.exists(_native.LIB_PATH):
        import __graft_entry__

        __graft_entry__.build()
    return _native.lib()


def test_header_symbols_are_exported(lib):
    names = declared_functions()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in vlgpu.h but not exported"


def test_binding_table_matches_header():
    from vectorlink_gpu import _native

    assert sorted(_native._SIGNATURES) == declared_functions()


def test_sentinels_match_reference_constants():
    from vectorlink_gpu.constants import MAXFLOAT, MAXINT, PRIMES_HOST

    text = open(HEADER).read()
    assert f"#define VL_MAXINT {MAXINT}" in text
    assert "#define VL_MAXFLOAT 3.4028e37f" in text and MAXFLOAT == 3.4028e37
    assert "#define VL_ERR_STATE (-4)" in text
    assert PRIMES_HOST.numel() == 965 and int(PRIMES_HOST[0]) == 10000349 and int(PRIMES_HOST[964]) == 1999


def test_host_side_validation(lib):
    from vectorlink_gpu import _native as nv

    one = C.c_void_p(256)  # never dereferenced: every call below is rejected on the host
    # insert that does not fit the queue
    rc = lib.vl_queue_insert(one, one, 4, 10, 8, one, one, 5, None, 0, None, None)
    assert rc == -1 and b"does not fit" in lib.vl_last_error()
    with pytest.raises(ValueError):
        nv.check(rc)
    # rows beyond what the LDS sort holds
    assert lib.vl_queue_sort(one, one, 4, 5000, None) == -1
    # negative sizes, null pointers
    assert lib.vl_gather_distances(one, -1, one, 10, 8, one, 4, one, None) == -1
    assert lib.vl_gather_distances(None, 3, one, 10, 8, one, 4, one, None) == -1
    assert lib.vl_prune(one, one, 10, 4, one, one, None) == -1  # in-place prune is refused
    # beam parameters: queue too small for one round of candidates, workspace too small
    p = nv.BeamParams(n_rows=10, dim=8, n_vectors=100, width=8, queue_capacity=20, queue_length=8, beam_size=4,
                      parallel_visit_count=4, visit_queue_factor=3, exclude_factor=5, speculative_readahead=5,
                      excl_cols=0, flags=0)
    assert lib.vl_beam_workspace_bytes(C.byref(p)) == -1
    p.queue_capacity = 8 + 32
    need = lib.vl_beam_workspace_bytes(C.byref(p))
    assert need > 0 and need % 256 == 0
    rc = lib.vl_closest_vectors(C.byref(p), one, one, one, one, one, None, one, need - 1, None)
    assert rc == -3 and b"workspace" in lib.vl_last_error()
    # exact kNN limits
    assert lib.vl_knn_workspace_bytes(10, 100, 8, 17) == -1
    assert lib.vl_knn_workspace_bytes(10, 100, 6, 10) == -1
    assert lib.vl_knn_workspace_bytes(10, 100, 8, 10) > 0
    # empty problems succeed without touching a device
    assert lib.vl_queue_sort(None, None, 0, 16, None) == 0
    assert lib.vl_search_from_seeds(None, 0, 8, None, 4, None, 10, 4, None, 10, None, None, None) == 0


def test_cpu_tensors_are_refused():
    import torch

    from vectorlink_gpu import Queue
    from vectorlink_gpu.kernels import calculate_distances

    v = torch.zeros((4, 8), dtype=torch.float32)
    b = torch.zeros((4, 2), dtype=torch.int32)
    with pytest.raises(RuntimeError):
        calculate_distances(v, b)
    q = Queue(2, 2, 6, device="cpu")
    with pytest.raises(RuntimeError):
        q.insert(torch.zeros((2, 2), dtype=torch.int32), torch.zeros((2, 2), dtype=torch.float32))


def test_library_is_not_older_than_its_sources():
    """The built library travels with the tree; one that predates an edit of its sources would be
    tested in their place."""
    from vectorlink_gpu import _native

    built = os.path.getmtime(_native.LIB_PATH)
    csrc = os.path.join(ROOT, "vectorlink-gpu_amd", "csrc")
    sources = [os.path.join(csrc, f) for f in os.listdir(csrc)] + [HEADER]
    stale = [os.path.basename(s) for s in sources if os.path.getmtime(s) > built]
    assert not stale, f"rebuild libvlgpu.so (python vectorlink-gpu_amd/build.py): newer sources {stale}"
