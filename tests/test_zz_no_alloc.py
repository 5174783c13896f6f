"""The entry point that allocates nothing (vl_closest_vectors_noalloc): a fixed number of launches on
the library's static scratch array, against vl_closest_vectors with a caller's workspace - same queues
bit for bit, on two calls in a row, the second smaller than the first."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda"


def test_no_alloc_entry_point_matches_the_workspace_one():
    print("vl_closest_vectors_noalloc: two calls in a row against vl_closest_vectors", flush=True)
    from vectorlink_gpu import Queue
    from vectorlink_gpu import _native as nv
    from vectorlink_gpu.ann import _beam_params, closest_vectors, excluding_self

    rng = np.random.default_rng(2024)
    n, dim, beam, bqf, pv = 5000, 48, 8, 2, 4
    v = rng.standard_normal((n, dim)).astype(np.float32)
    v /= np.linalg.norm(v, axis=1, keepdims=True)
    c = dict(orc.DEFAULT_CONFIG, beam_size=beam, beam_queue_factor=bqf, parallel_visit_count=pv)
    ql = beam * bqf
    gv = torch.from_numpy(v).to(DEV)
    gb = torch.from_numpy(orc.generate_circulant_beams(n, orc.primes(ql))).to(DEV)
    gd = torch.from_numpy(orc.calculate_distances(v, gb.cpu().numpy())).to(DEV)
    status = torch.full((2,), -7, dtype=torch.int32, device=DEV)

    def seeded(lo, hi):
        q = Queue(hi - lo, ql, ql + ql * pv)
        q.insert(gb[lo:hi], gd[lo:hi])
        return q

    for (lo, hi) in ((100, 3100), (4000, 4700)):          # the second call is smaller than the first
        want = seeded(lo, hi)
        t_want = closest_vectors(gv[lo:hi], want, gv, gb, c, excluding_self(lo, hi))
        got = seeded(lo, hi)
        excl = excluding_self(lo, hi)
        queries = gv[lo:hi].contiguous()
        p = _beam_params(hi - lo, dim, n, ql, got, c, 1)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        rc = nv.lib().vl_closest_vectors_noalloc(ctypes.byref(p), nv.ptr(queries), nv.ptr(gv), nv.ptr(gb),
                                                 nv.ptr(got.indices), nv.ptr(got.distances), nv.ptr(excl),
                                                 t_want + 7, nv.ptr(status), nv.stream())
        assert rc == 0, nv.lib().vl_last_error()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert status.tolist() == [1, t_want]
        assert torch.equal(got.indices[:, :ql], want.indices[:, :ql])
        assert torch.equal(got.distances[:, :ql].view(torch.int32), want.distances[:, :ql].view(torch.int32))
        # too few launches: reported as unfinished
        short = seeded(lo, hi)
        p = _beam_params(hi - lo, dim, n, ql, short, c, 1)
        rc = nv.lib().vl_closest_vectors_noalloc(ctypes.byref(p), nv.ptr(queries), nv.ptr(gv), nv.ptr(gb),
                                                 nv.ptr(short.indices), nv.ptr(short.distances), nv.ptr(excl),
                                                 3, nv.ptr(status), nv.stream())
        assert rc == 0
        torch.cuda.synchronize()
        assert status.tolist() == [0, 3]

    # a batch beyond the static array is refused on the host, with the sizes in the message
    big = seeded(0, 8)
    p = _beam_params(400_000, dim, n, ql, big, c, 0)
    rc = nv.lib().vl_closest_vectors_noalloc(ctypes.byref(p), nv.ptr(gv), nv.ptr(gv), nv.ptr(gb), nv.ptr(big.indices),
                                             nv.ptr(big.distances), None, 10, nv.ptr(status), nv.stream())
    assert rc == -1 and b"static array" in nv.lib().vl_last_error()
