"""Batched fixed-capacity sorted queues (reference: vectorlink_gpu/queue.py)."""
from typing import Optional

import torch
from torch import Tensor

from . import _native as nv
from .constants import DEVICE, MAXFLOAT, MAXINT
from .utils import queue_sort  # noqa: F401  (re-exported like the reference's module-level queue_sort)


class Queue:
    def __init__(self, num_queues: int, queue_length: int, capacity: int, device=DEVICE):
        assert queue_length < capacity  # queue.py:23
        self.length = queue_length
        self.indices = torch.full((num_queues, capacity), MAXINT, dtype=torch.int32, device=device)
        self.distances = torch.full((num_queues, capacity), MAXFLOAT, dtype=torch.float32, device=device)

    def initialize_from_queue(self, queue):
        """Take over the head of another queue: its first min(length, other.length) slots (reference queue.py:30-35)."""
        n = min(queue.length, self.length)
        self.indices[:, :n] = queue.indices[:, :n]
        self.distances[:, :n] = queue.distances[:, :n]

    def insert(
        self,
        vector_id_batch: Tensor,
        distances_batch: Tensor,
        exclude: Optional[Tensor] = None,  # formatted like [[0,MAXINT...],[1],[2]]
        output_update: bool = False,
    ):
        """queue.py:37-61 as one kernel: copy to the tail, punch out exclusions,
        order by (distance, id), drop neighbouring duplicates."""
        (batches, size_per_batch) = vector_id_batch.size()
        (rows, capacity) = self.indices.size()
        assert batches == rows and vector_id_batch.size() == distances_batch.size()
        assert vector_id_batch.dtype == torch.int32 and distances_batch.dtype == torch.float32
        ids = vector_id_batch.contiguous()
        dists = distances_batch.contiguous()
        excl = None
        if exclude is not None:
            assert exclude.dtype == torch.int32 and exclude.size(0) == rows
            excl = exclude.contiguous()
        nv.require_gpu(self.indices, self.distances, ids, dists, excl)
        mask = None
        if output_update:
            mask = torch.empty((rows, self.length), dtype=torch.uint8, device=self.indices.device)
        nv.check(nv.lib().vl_queue_insert(
            nv.ptr(self.indices), nv.ptr(self.distances), rows, capacity, self.length, nv.ptr(ids), nv.ptr(dists),
            size_per_batch, nv.ptr(excl), 0 if excl is None else excl.size(1), nv.ptr(mask), nv.stream()))
        if output_update:
            return mask.to(torch.bool)
        return None

    def print(self, tail: Optional[bool] = False):
        """Dump the first `length` slots, and with tail=True the slots behind them."""
        for part in ((slice(0, self.length),) + ((slice(self.length, None),) if tail else ())):
            if part.start:
                print("-" * 16)
            print(self.indices[:, part])
            print(self.distances[:, part])

    def pop_n_ids(self, n: int):
        """queue.py:87-95"""
        take = min(self.length, n)
        (rows, capacity) = self.indices.size()
        nv.require_gpu(self.indices)
        out = torch.empty((rows, take), dtype=torch.int32, device=self.indices.device)
        nv.check(nv.lib().vl_queue_pop(nv.ptr(self.indices), nv.ptr(self.distances), rows, capacity, take,
                                       nv.ptr(out), nv.stream()))
        return out

    def size(self):
        return self.indices.size()
