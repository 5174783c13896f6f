"""Seeded synthetic workloads: unit-norm float32 vectors on the CPU generator, so
the same bits are available to a CPU checker and to the GPU (the reference's
own generator is normalize(randn(N, D)), utils.py:15-19 - workload "iid")."""
from typing import Dict, Tuple

import torch
from torch import Tensor

CPU = torch.device("cpu")  # every draw names its device: a caller may have changed torch's default

# name -> parameters.  beam_size = graph degree, beam_queue_factor = build queue / degree,
# recall_search_queue_factor = search queue / degree; the remaining knobs are the class defaults.
WORKLOADS: Dict[str, Dict] = {
    "iid-4k-128": dict(n=4096, dim=128, kind="iid", seed=0, queries=256, beam_size=32, beam_queue_factor=2,
                       recall_search_queue_factor=2),
    "mix-1m-128": dict(n=1_000_000, dim=128, kind="mixture", centres=1024, sigma=0.1, seed=1, queries=10_000,
                       beam_size=32, beam_queue_factor=2, recall_search_queue_factor=2),
    "mix-1m-768": dict(n=1_000_000, dim=768, kind="mixture", centres=4096, sigma=0.15, seed=2, queries=10_000,
                       beam_size=64, beam_queue_factor=2, recall_search_queue_factor=2),
    # cluster sizes follow rank^-1.1 and 2 % of the rows are exact copies of other rows
    "zipf-20m-384": dict(n=20_000_000, dim=384, kind="zipf", centres=16_384, sigma=0.15, zipf_s=1.1, duplicates=0.02,
                         seed=3, queries=50_000, beam_size=48, beam_queue_factor=2, recall_search_queue_factor=2),
    "mix-10m-1536": dict(n=10_000_000, dim=1536, kind="mixture", centres=8192, sigma=0.2, seed=4, queries=100_000,
                         beam_size=64, beam_queue_factor=2, recall_search_queue_factor=2),
}


def _normalise_(x: Tensor) -> Tensor:
    return torch.nn.functional.normalize(x, dim=1, out=x)


def _mixture(gen: torch.Generator, centres: Tensor, count: int, sigma: float, chunk: int = 100_000,
             weights: Tensor = None) -> Tensor:
    dim = centres.size(1)
    out = torch.empty((count, dim), dtype=torch.float32, device=CPU)
    if weights is None:
        assign = torch.randint(0, centres.size(0), (count,), generator=gen, device=CPU)
    else:
        assign = torch.multinomial(weights, count, replacement=True, generator=gen)
    for s in range(0, count, chunk):
        e = min(s + chunk, count)
        noise = torch.randn((e - s, dim), generator=gen, dtype=torch.float32, device=CPU)
        out[s:e] = centres[assign[s:e]] + sigma * noise
        _normalise_(out[s:e])
    return out


def make(name: str, n: int = None, queries: int = None, centres: int = None) -> Tuple[Tensor, Tensor, Dict]:
    """Returns (vectors [n, dim], queries [q, dim], parameters) as CPU float32 tensors.
    n / queries / centres override the workload's sizes (the draw order is fixed: centres, base
    set, duplicate rows, queries)."""
    w = dict(WORKLOADS[name])
    if n is not None:
        w["n"] = n
    if queries is not None:
        w["queries"] = queries
    if centres is not None:
        w["centres"] = centres
    gen = torch.Generator(device=CPU).manual_seed(w["seed"])
    if w["kind"] == "iid":
        base = _normalise_(torch.randn((w["n"], w["dim"]), generator=gen, dtype=torch.float32, device=CPU))
        q = _normalise_(torch.randn((w["queries"], w["dim"]), generator=gen, dtype=torch.float32, device=CPU))
    elif w["kind"] == "zipf":
        centres = torch.randn((w["centres"], w["dim"]), generator=gen, dtype=torch.float32, device=CPU)
        weights = torch.arange(1, w["centres"] + 1, dtype=torch.float64, device=CPU).pow(-w["zipf_s"])
        base = _mixture(gen, centres, w["n"], w["sigma"], weights=weights)
        copies = int(w["n"] * w["duplicates"])
        dst = torch.randperm(w["n"], generator=gen, device=CPU)[:copies]
        src = torch.randint(0, w["n"], (copies,), generator=gen, device=CPU)
        base[dst] = base[src]
        q = _mixture(gen, centres, w["queries"], w["sigma"], weights=weights)
    else:
        centres = torch.randn((w["centres"], w["dim"]), generator=gen, dtype=torch.float32, device=CPU)
        base = _mixture(gen, centres, w["n"], w["sigma"])
        q = _mixture(gen, centres, w["queries"], w["sigma"])
    return base, q, w


def ann_kwargs(w: Dict) -> Dict:
    return dict(beam_size=w["beam_size"], beam_queue_factor=w["beam_queue_factor"],
                recall_search_queue_factor=w["recall_search_queue_factor"])
