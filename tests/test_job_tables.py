"""Host logic of the job tables the model-level API writes (no GPU: the entry point is a
stand-in that reads the table it is handed)."""
import ctypes

import torch

from compressed_tensors_amd import _lib
from compressed_tensors_amd.compressors.job_tables import (
    WeightJobTable, module_chunks, run_table, slab_outputs,
)


class _Plan:
    def __init__(self, **fields):
        self.qp = _lib.QParams()
        for k, v in fields.items():
            setattr(self.qp, k, v)


def _capture(seen):
    def entry(jobs, n, *rest):
        seen.append(([(jobs[i].src, jobs[i].dst, jobs[i].rows, jobs[i].cols, jobs[i].dense_dtype,
                       jobs[i].qp.scale, jobs[i].qp.zero_point, jobs[i].qp.global_scale,
                       jobs[i].qp.s_cols, jobs[i].qp.blk_cols, jobs[i].qp.num_bits) for i in range(n)], rest))
        return 0
    return entry


def test_rows_and_templates_reach_the_entry_point():
    table = WeightJobTable()
    a = table.add_template("a", _Plan(s_cols=32, blk_cols=128, num_bits=4, scale=111, zero_point=222, global_scale=333))
    b = table.add_template("b", _Plan(s_cols=1, blk_cols=4096, num_bits=8))
    assert (table.template("a"), table.template("b"), table.template("c"), table.n_templates) == (a, b, -1, 2)
    table.add(1000, 2000, 8, 4096, 7, a, 3000)
    table.add(1001, 2001, 16, 4096, 7, b, 3001, 4001, 5001)
    table.add(1002, 2002, 24, 4096, 7, a, 3002, 4002)
    seen = []
    table.launch(_capture(seen), 77)
    rows, rest = seen[0]
    assert rest == (77,)
    # addresses come from the rows, never from the plan the template was made of
    assert rows == [(1000, 2000, 8, 4096, 7, 3000, None, None, 32, 128, 4),
                    (1001, 2001, 16, 4096, 7, 3001, 4001, 5001, 1, 4096, 8),
                    (1002, 2002, 24, 4096, 7, 3002, 4002, None, 32, 128, 4)]
    assert len(table) == 0
    table.launch(_capture(seen), 77)  # nothing added: no call
    assert len(seen) == 1


def test_a_template_cannot_carry_a_column_group_table():
    import pytest

    with pytest.raises(ValueError):
        WeightJobTable().add_template("g", _Plan(col_group=1234))


def test_the_qdq_job_shares_the_layout():
    table = WeightJobTable(_lib.QdqJob)
    t = table.add_template("k", _Plan(num_bits=8))
    table.add(1, 2, 3, 4, 5, t, 6, 0, 0, 9)
    got = []

    def entry(jobs, n, do_q, do_dq, stream):
        got.append((jobs[0].x, jobs[0].out, jobs[0].rows, jobs[0].cols, jobs[0].x_dtype, jobs[0].out_dtype,
                    jobs[0].qp.scale, do_q, do_dq, stream))
        return 0

    table.launch(entry, 1, 0, 99)
    assert got == [(1, 2, 3, 4, 5, 9, 6, 1, 0, 99)]


def test_chunks_start_short():
    assert list(module_chunks(0)) == []
    assert list(module_chunks(10)) == [(0, 10)]
    assert list(module_chunks(224)) == [(0, 16), (16, 48), (48, 112), (112, 176), (176, 224)]


def test_outputs_of_one_shape_share_allocations():
    shapes = [(4, 64)] * 5 + [(3, 5)] * 2 + [(4, 64)]
    outs = slab_outputs(shapes, torch.float32, torch.device("cpu"))
    assert [tuple(t.shape) for t in outs] == shapes
    same = [t for t, s in zip(outs, shapes) if s == (4, 64)]
    assert len({t.untyped_storage().data_ptr() for t in same}) == 1  # one allocation, six slices
    assert len({t.data_ptr() for t in same}) == 6 and all(t.is_contiguous() for t in same)
    assert all(t.data_ptr() % 256 == same[0].data_ptr() % 256 for t in same)
    odd = [t for t, s in zip(outs, shapes) if s == (3, 5)]  # 60 bytes: slices would lose their alignment
    assert odd[0].untyped_storage().data_ptr() != odd[1].untyped_storage().data_ptr()


class _Spec:
    """takes even records, refuses odd ones"""
    job_struct = _lib.WeightJob

    def key(self, rec):
        return None if rec % 2 else ("k", rec % 4)

    def out_spec(self, rec):
        return (2, 128), torch.float32, torch.device("cpu")

    def plan(self, rec):
        return _Plan(num_bits=rec % 4 + 1)

    def row(self, rec, out):
        return (1000 + rec, out.data_ptr(), 2, 128, 1, 7 + 10 * rec, 0, 0, 0)


class _Owner:
    pass


def test_the_engine_streams_records_into_calls(monkeypatch):
    monkeypatch.setattr(_lib, "stream_of", lambda device: 5)
    seen = []
    outs = run_table(_Owner(), (r for r in range(100)), _Spec(), _capture(seen))
    assert len(outs) == 100
    assert all((o is None) == bool(r % 2) for r, o in enumerate(outs))
    sizes = [len(rows) for rows, _ in seen]
    assert sizes == [16, 32, 2]  # 50 records taken: short calls first
    flat = [row for rows, _ in seen for row in rows]
    assert [row[0] - 1000 for row in flat] == list(range(0, 100, 2))   # in order
    assert all(row[5] == 7 + 10 * (row[0] - 1000) and row[10] == (row[0] - 1000) % 4 + 1
               for row in flat)  # own scale, own template
    assert all(rest == (5,) for _, rest in seen)
    assert [row[1] for row in flat] == [outs[row[0] - 1000].data_ptr() for row in flat]
