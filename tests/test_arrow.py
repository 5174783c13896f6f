"""Arrow <-> tensor conversions on the CPU, and the index round trip on the GPU."""
import numpy as np
import pyarrow as pa
import pytest
import torch

from vectorlink_gpu.datafusion import dataframe_to_tensor, tensor_to_arrow


def test_tensor_to_arrow_and_back():
    t = torch.arange(12, dtype=torch.float32).reshape(4, 3)
    arr = tensor_to_arrow(t)
    assert isinstance(arr, pa.FixedSizeListArray) and arr.type.list_size == 3 and len(arr) == 4
    assert arr.to_pylist() == t.tolist()
    back = torch.empty((4, 3), dtype=torch.float32)
    dataframe_to_tensor(arr, back)
    assert torch.equal(back, t)
    ids = torch.tensor([[1, 2], [3, 4]], dtype=torch.int32)
    assert tensor_to_arrow(ids).to_pylist() == [[1, 2], [3, 4]]
    with pytest.raises(ValueError):
        tensor_to_arrow(ids.double())


def test_dataframe_to_tensor_sources():
    rows = np.arange(20, dtype=np.float32).reshape(5, 4)
    var = pa.array(rows.tolist(), type=pa.list_(pa.float32()))        # variable-size list type, fixed lengths
    fixed = pa.FixedSizeListArray.from_arrays(pa.array(rows.reshape(-1)), 4)
    table = pa.table({"embedding": pa.chunked_array([var[:2], var[2:]]), "other": fixed})
    for src, col in [(table, "embedding"), (table, "other"), (table.to_batches()[0], 0), (var, 0),
                     (pa.RecordBatchReader.from_batches(table.schema, table.to_batches()), "embedding")]:
        out = torch.empty((len(src) if not isinstance(src, pa.RecordBatchReader) else 5, 4), dtype=torch.float32)
        if isinstance(src, pa.RecordBatch):
            out = torch.empty((src.num_rows, 4), dtype=torch.float32)
        dataframe_to_tensor(src, out, col)
        assert np.array_equal(out.numpy(), rows[:out.shape[0]])

    class FakeDataFusionFrame:  # duck-typed like datafusion.DataFrame.execute_stream()
        class _B:
            def __init__(self, b):
                self.b = b

            def to_pyarrow(self):
                return self.b

        def execute_stream(self):
            return [self._B(b) for b in table.to_batches()]

    out = torch.empty((5, 4), dtype=torch.float32)
    dataframe_to_tensor(FakeDataFusionFrame(), out)
    assert np.array_equal(out.numpy(), rows)
    with pytest.raises(ValueError):
        dataframe_to_tensor(table, torch.empty((4, 4), dtype=torch.float32), "embedding")   # too many rows
    with pytest.raises(ValueError):
        dataframe_to_tensor(table, torch.empty((5, 3), dtype=torch.float32), "embedding")   # wrong width
    ragged = pa.array([[1.0, 2.0], [3.0]], type=pa.list_(pa.float32()))
    with pytest.raises(ValueError):
        dataframe_to_tensor(ragged, torch.empty((2, 2), dtype=torch.float32))


@pytest.mark.gpu
def test_index_round_trip_through_arrow():
    from vectorlink_gpu import ANN

    rng = np.random.default_rng(3)
    v = rng.standard_normal((900, 16)).astype(np.float32)
    v /= np.linalg.norm(v, axis=1, keepdims=True)
    kw = dict(beam_queue_factor=2, recall_search_queue_factor=2, batch_size=400, optimization_loops=1)
    ann = ANN(torch.from_numpy(v).cuda(), beam_size=8, keep_queues=True, **kw)
    table = ann.to_arrow()
    assert table.schema.names == ["vector_id", "embedding", "beams", "distances"] and table.num_rows == 900
    shuffled = table.take(pa.array(rng.permutation(900)))            # load_from_dataframe orders by vector_id
    again = ANN.load_from_dataframe(shuffled, **kw)
    assert torch.equal(again.vectors, ann.vectors) and torch.equal(again.beams, ann.beams)
    assert torch.equal(again.distances, ann.distances)
    q = torch.from_numpy(v[:50]).cuda()
    a, b = ann.search(q), again.search(q)
    assert torch.equal(a.indices[:, :a.length], b.indices[:, :b.length])
    no_d = ANN.load_from_dataframe(shuffled.drop_columns(["distances"]), **kw)   # distances recomputed (ann.py:393-394)
    assert torch.equal(no_d.distances, ann.distances)
    # clusters(): the search queues the build ended with (full build-queue width), None unless kept
    queues = ann.clusters()
    assert queues.indices.shape == (900, 17) and queues.length == 16
    assert torch.equal(queues.indices[:, :8], ann.beams)
    assert again.clusters() is None
