"""The committed fixture tests/golden/ann_small.npz: the oracle still reproduces it (CPU), and
the HIP path matches it (GPU) without the oracle being involved."""
import importlib.util
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURE = os.path.join(HERE, "golden", "ann_small.npz")


def _maker():
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(HERE, "golden", "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_oracle_reproduces_the_fixture():
    mk = _maker()
    g = np.load(FIXTURE)
    v, q = mk.inputs()
    assert np.array_equal(v, g["vectors"]) and np.array_equal(q, g["queries"])
    out = mk.outputs(v, q)
    for name, want in out.items():
        got = g[name]
        if want.dtype == np.float32:
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), name
        else:
            assert np.array_equal(got, want), name


@pytest.mark.gpu
def test_hip_path_matches_the_fixture():
    import torch

    from vectorlink_gpu import ANN
    from vectorlink_gpu.kernels import optimize_graph, prune_

    mk = _maker()
    g = np.load(FIXTURE)
    kw = {k: mk.CONFIG[k] for k in ("beam_size", "beam_queue_factor", "recall_search_queue_factor", "batch_size",
                                    "optimization_loops")}
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    ann = ANN(dev(g["vectors"]), **kw)
    assert np.array_equal(ann.beams.cpu().numpy(), g["beams"])
    assert np.allclose(ann.distances.cpu().numpy(), g["distances"], rtol=1e-5, atol=1e-6)
    assert np.array_equal(ann.distances.cpu().numpy().view(np.uint32), g["distances"].view(np.uint32))
    res = ann.search(dev(g["queries"]))
    L = res.length
    assert np.array_equal(res.indices.cpu().numpy()[:, :L], g["search_ids"])
    assert np.allclose(res.distances.cpu().numpy()[:, :L], g["search_distances"], rtol=1e-5, atol=1e-6)
    pb, pd = prune_(dev(g["wide"]), dev(g["wide_distances"]))
    assert np.array_equal(pb.cpu().numpy(), g["pruned"])
    assert np.array_equal(pd.cpu().numpy().view(np.uint32), g["pruned_distances"].view(np.uint32))
    assert np.array_equal(optimize_graph(dev(g["wide"]), mk.CONFIG["beam_size"]).cpu().numpy(), g["optimized"])
