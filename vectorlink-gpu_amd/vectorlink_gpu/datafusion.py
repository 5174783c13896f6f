"""Arrow in and out of GPU tensors (reference: vectorlink_gpu/datafusion.py).

The reference streams a DataFusion DataFrame into a preallocated CUDA tensor
through Numba (datafusion.py:36-52) and turns a tensor into an Arrow array
(datafusion.py:55-56).  Here the same two directions work on pyarrow objects
(Table, RecordBatch, RecordBatchReader, ChunkedArray, Array) and on anything
that offers DataFusion's `execute_stream()` / `to_arrow_table()`; DataFusion
itself is not required.  Object-store session builders are not provided.
"""
from typing import Iterable

import numpy as np
import pyarrow as pa
import torch
from torch import Tensor


def dtype_to_arrow(dtype):
    """reference datafusion.py:27-33 (there: dtype -> ctypes)"""
    if dtype == torch.float32:
        return pa.float32()
    if dtype == torch.int32:
        return pa.int32()
    raise ValueError(f"i don't know what a {dtype} is")


def tensor_to_arrow(tensor: Tensor) -> pa.Array:
    """reference datafusion.py:55-56: one list per row; here a FixedSizeListArray that
    shares the (host copy of the) tensor's buffer instead of building Python lists"""
    assert tensor.dim() == 2
    host = tensor.detach().cpu().contiguous().numpy()
    flat = pa.array(host.reshape(-1), type=dtype_to_arrow(tensor.dtype))
    return pa.FixedSizeListArray.from_arrays(flat, host.shape[1])


def _column_batches(source, column) -> Iterable[pa.Array]:
    if isinstance(source, (pa.Array, pa.ChunkedArray)):
        chunks = source.chunks if isinstance(source, pa.ChunkedArray) else [source]
        yield from chunks
        return
    if isinstance(source, pa.RecordBatch):
        yield source.column(column)
        return
    if isinstance(source, pa.Table):
        yield from source.column(column).chunks
        return
    if hasattr(source, "execute_stream"):  # a DataFusion DataFrame
        for batch in source.execute_stream():
            yield batch.to_pyarrow().column(column)
        return
    if hasattr(source, "read_next_batch") or isinstance(source, pa.RecordBatchReader):
        for batch in source:
            yield batch.column(column)
        return
    raise TypeError(f"cannot read Arrow batches from {type(source)}")


def _list_values(arr: pa.Array, width: int, np_dtype) -> np.ndarray:
    """rows of a list / large_list / fixed_size_list array as a [len, width] numpy view"""
    if arr.null_count:
        raise ValueError("null rows are not supported")
    if pa.types.is_fixed_size_list(arr.type):
        if arr.type.list_size != width:
            raise ValueError(f"rows of {arr.type.list_size} values, expected {width}")
        values = arr.flatten()
    elif pa.types.is_list(arr.type) or pa.types.is_large_list(arr.type):
        offsets = arr.offsets.to_numpy()
        if len(arr) and not np.all(np.diff(offsets) == width):
            raise ValueError(f"every row must hold {width} values")
        values = arr.flatten()
    else:
        raise TypeError(f"expected a list column, got {arr.type}")
    if values.null_count:
        raise ValueError("null values are not supported")
    out = values.to_numpy(zero_copy_only=False)
    if out.dtype != np_dtype:
        out = out.astype(np_dtype)
    return out.reshape(len(arr), width)


def dataframe_to_tensor(source, tensor: Tensor, column=0):
    """reference datafusion.py:36-52: fill the preallocated [N, width] tensor with the
    rows of a list column, batch by batch, in the order the source yields them
    (the caller sorts, as the reference asks).  Host batches are staged through
    one pinned buffer when the tensor lives on the GPU."""
    assert tensor.dim() == 2 and tensor.is_contiguous()
    np_dtype = {torch.float32: np.float32, torch.int32: np.int32}[tensor.dtype]
    (count, width) = tensor.size()
    offset = 0
    for arr in _column_batches(source, column):
        rows = _list_values(arr, width, np_dtype)
        if offset + len(rows) > count:
            raise ValueError("the source holds more rows than the tensor")
        rows = np.ascontiguousarray(rows)
        chunk = torch.from_numpy(rows if rows.flags.writeable else rows.copy())
        if tensor.is_cuda:
            chunk = chunk.pin_memory()
        tensor[offset:offset + len(rows)].copy_(chunk, non_blocking=False)
        offset += len(rows)
    if offset != count:
        raise ValueError(f"the source held {offset} rows, the tensor expects {count}")
    return tensor
