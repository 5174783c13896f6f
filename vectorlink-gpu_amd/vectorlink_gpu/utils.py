"""Host-side helpers with the reference's names (vectorlink_gpu/utils.py)."""
import torch
from torch import Tensor

from . import _native as nv
from .constants import DEVICE, MAXINT, primes_on
from .kernels import dedup_tensor_, index_sort_, queue_sort_


def generate_random_vectors(number_of_vectors: int, dimensions: int = 1536, device=DEVICE) -> Tensor:
    """reference utils.py:15-19"""
    return torch.nn.functional.normalize(
        torch.randn(number_of_vectors, dimensions, dtype=torch.float32, device=device), dim=1)


def primes(size: int, device=DEVICE) -> Tensor:
    """reference utils.py:22-23"""
    assert 0 <= size <= 965, "the prime table has 965 entries"
    return primes_on(device).narrow(0, 0, size)


def _circulants(rows: int, modulus: int, p: Tensor) -> Tensor:
    assert p.dtype == torch.int32 and p.dim() == 1
    nv.require_gpu(p)
    p = p.contiguous()
    out = torch.empty((rows, p.size(0)), dtype=torch.int32, device=p.device)
    nv.check(nv.lib().vl_circulants(nv.ptr(out), rows, 0, modulus, nv.ptr(p), p.size(0), nv.stream()))
    return out


def generate_queue_circulants(batch_size: int, num_vecs: int, primes: Tensor) -> Tensor:
    """reference utils.py:26-32: row b = sort(b + primes) % num_vecs"""
    return _circulants(batch_size, num_vecs, primes)


def generate_circulant_beams(num_vecs: int, primes: Tensor) -> Tensor:
    """reference utils.py:35-41: row i = sort(i + primes) % num_vecs"""
    return _circulants(num_vecs, num_vecs, primes)


def index_sort(beams: Tensor, beam_distances: Tensor):
    """reference utils.py:44-53 (returns new tensors ordered by (distance, id))"""
    ns = beams.contiguous().clone()
    nds = beam_distances.contiguous().clone()
    index_sort_(ns, nds)
    return (ns, nds)


def queue_sort(beams: Tensor, beam_distances: Tensor):
    """reference utils.py:56-58 / queue.py:15-18"""
    ns = beams.contiguous().clone()
    nds = beam_distances.contiguous().clone()
    queue_sort_(ns, nds)
    return (ns, nds)


def add_new_to_seen_(seen: Tensor, indices: Tensor):
    """reference utils.py:61-82: returns None when no column is free in every row"""
    assert seen.dtype == torch.int32 and seen.is_contiguous()
    indices = indices.contiguous()
    nv.require_gpu(seen, indices)
    import ctypes

    status = ctypes.c_int(0)
    ws = torch.empty(2, dtype=torch.int32, device=seen.device)
    nv.check(nv.lib().vl_seen_add(nv.ptr(seen), seen.size(0), seen.size(1), nv.ptr(indices), indices.size(1),
                                  nv.ptr(ws), ctypes.byref(status), nv.stream()))
    return seen if status.value else None


def dedup_sort(tensor: Tensor):
    """reference utils.py:85-89"""
    (tensor, _) = tensor.sort()
    tensor = tensor.contiguous()
    dedup_tensor_(tensor)
    (tensor, _) = tensor.sort()
    return tensor
