"""Job tables of the many-weight entry points, filled a column at a time.

A model has hundreds of weights and a handful of distinct (shape, dtype, scheme)
combinations.  What `build_qparams` derives for a weight depends on that combination
only, apart from three addresses; a table of `ctmi_weight_job` is therefore written
as numpy columns (addresses and sizes from Python lists, the scale-grid description
gathered from one template per combination) instead of field by field, which keeps
the host side of `compress_model` / `decompress_model` shorter than the kernels
they enqueue.
"""
import ctypes
from typing import Dict, List, Tuple

import numpy as np
import torch

from compressed_tensors_amd import _lib

__all__ = ["WeightJobTable", "slab_outputs", "module_table", "module_chunks", "args_key", "FLOAT_DTYPES",
           "run_table", "on_gpu"]

_QP = np.dtype(_lib.QParams)
assert _QP.itemsize == ctypes.sizeof(_lib.QParams)

FLOAT_DTYPES = (torch.bfloat16, torch.float16, torch.float32)
_CHUNK_MODULES = 64   # modules per call of the C ABI on the module pathways

_SLAB_BYTES = 1 << 30   # outputs of one shape share an allocation up to this size
_ALIGN = 256            # ... if each of them keeps this alignment inside it


class WeightJobTable:
    """Rows are added with `add`; `launch` writes them into an array of `job_struct` and hands
    it to a many-weight entry point.  `add_template` registers the part of a job's qparams
    that holds no scale, zero-point or global-scale address (as `build_qparams` made it for
    one weight of the combination).

    job_struct: `ctmi_weight_job` (source, destination, rows, cols, dtype of the dense side,
    reserved, qparams) or `ctmi_qdq_job`, which has the same layout with the dtypes of input
    and output in the two 32-bit members."""

    def __init__(self, job_struct=_lib.WeightJob):
        self._job = np.dtype(job_struct)
        assert self._job.itemsize == ctypes.sizeof(job_struct)
        names = self._job.names
        assert len(names) == 7 and names[2:4] == ("rows", "cols") and names[6] == "qp"
        self._f_src, self._f_dst, self._f_dtype, self._f_dtype2 = names[0], names[1], names[4], names[5]
        self._job_ptr = ctypes.POINTER(job_struct)
        self._templates: List[np.ndarray] = []
        self._template_of: Dict[Tuple, int] = {}
        self.clear()

    def clear(self):
        """drop the rows added since the last launch"""
        self.src, self.dst, self.rows, self.cols, self.dense_dtype = [], [], [], [], []
        self.scale, self.zero_point, self.which = [], [], []
        self.global_scale, self.second_dtype = [], []

    @property
    def n_templates(self) -> int:
        return len(self._templates)

    def template(self, key) -> int:
        """index of the template registered under `key`, or -1"""
        return self._template_of.get(key, -1)

    def add_template(self, key, plan) -> int:
        qp = np.frombuffer(bytes(plan.qp), dtype=_QP).copy()
        if int(qp["col_group"][0]):
            raise ValueError("a template cannot hold the address of a column-group table")
        qp["scale"] = 0
        qp["zero_point"] = 0
        qp["global_scale"] = 0
        self._templates.append(qp)
        self._stacked = np.concatenate(self._templates)
        self._template_of[key] = len(self._templates) - 1
        return len(self._templates) - 1

    def add(self, src: int, dst: int, rows: int, cols: int, dense_dtype: int, which: int,
            scale: int, zero_point: int = 0, global_scale: int = 0, second_dtype: int = 0) -> None:
        """dense_dtype / second_dtype: the two 32-bit members of the job (ctmi_weight_job: dtype
        of the dense side, reserved; ctmi_qdq_job: dtype of the input, of the output)"""
        self.src.append(src)
        self.dst.append(dst)
        self.rows.append(rows)
        self.cols.append(cols)
        self.dense_dtype.append(dense_dtype)
        self.second_dtype.append(second_dtype)
        self.which.append(which)
        self.scale.append(scale)
        self.zero_point.append(zero_point)
        self.global_scale.append(global_scale)

    def __len__(self):
        return len(self.src)

    def launch(self, entry, *args) -> None:
        """one call of `entry(jobs, n, *args)` for the rows added since the last launch"""
        n = len(self.src)
        if n == 0:
            return
        tab = np.zeros(n, self._job)
        tab[self._f_src] = self.src
        tab[self._f_dst] = self.dst
        tab["rows"] = self.rows
        tab["cols"] = self.cols
        tab[self._f_dtype] = self.dense_dtype
        tab[self._f_dtype2] = self.second_dtype
        qp = self._stacked[self.which]
        qp["scale"] = self.scale
        qp["zero_point"] = self.zero_point
        qp["global_scale"] = self.global_scale
        tab["qp"] = qp
        self.clear()
        # the entry points read the table before they return: it need not outlive the call
        _lib.check(entry(ctypes.cast(tab.ctypes.data, self._job_ptr), n, *args))


_RAMP = (16, 32)  # the first calls are short: the GPU starts while the later rows are written


def module_chunks(n):
    """(lo, hi) ranges over n weights: 16, 32, then 64 at a time"""
    at, k = 0, 0
    while at < n:
        size = _RAMP[k] if k < len(_RAMP) else _CHUNK_MODULES
        yield at, min(at + size, n)
        at += size
        k += 1


def module_table(compressor, job_struct=_lib.WeightJob) -> WeightJobTable:
    """the compressor's job table for the module pathways: its templates (the pointer-free
    part of a weight's qparams per shape / dtype / scheme) stay valid from call to call"""
    table = compressor.__dict__.get("_table")
    if table is None or table.n_templates > 512:
        table = compressor.__dict__["_table"] = WeightJobTable(job_struct)
    table.clear()  # rows a failed call may have left behind
    return table


def args_key(args):
    """what of a QuantizationArgs decides a weight's qparams plan"""
    return (args.num_bits, args.type, args.symmetric, args.strategy, args.group_size,
            None if args.block_structure is None else tuple(args.block_structure))


def on_gpu(t, device=None) -> bool:
    """is `t` a contiguous tensor on a GPU (on `device`, if given)?"""
    return (t is not None and t.device.type == "cuda" and t.is_contiguous()
            and (device is None or t.device == device))


def run_table(compressor, recs, spec, entry, *entry_args) -> list:
    """The many-weight call `entry(jobs, n, *entry_args, stream)` for the records of `recs`
    that `spec` takes; returns one output tensor per record, None for those it does not take
    (the caller treats them one by one).  `spec` describes a format and direction:
      spec.job_struct       ctmi_weight_job or ctmi_qdq_job
      spec.key(rec)         template key (what decides the qparams besides addresses), or None
      spec.out_spec(rec)    (shape, dtype, device) of the output
      spec.plan(rec)        the QPlan of build_qparams for this record (made once per key)
      spec.row(rec, out)    (src, dst, rows, cols, dtype code, scale, zero_point, global_scale,
                             second dtype code): addresses and sizes of the job
    Outputs of one shape share allocations; calls are short at first, so that the GPU starts
    while later rows are still being written."""
    outs: list = []
    pending: Dict[Tuple, List] = {}   # (dtype, device) of the outputs -> rows waiting for their call
    calls: Dict[Tuple, int] = {}      # ... -> calls made so far (the first ones are short)
    table = None

    def flush(group):
        nonlocal table
        part = pending.pop(group)
        if table is None:
            table = module_table(compressor, spec.job_struct)
        dtype, device = group
        slabs = slab_outputs([shape for _, _, _, shape in part], dtype, device)
        for (i, rec, key, _), out in zip(part, slabs):
            which = table.template(key)
            if which < 0:
                which = table.add_template(key, spec.plan(rec))
            src, dst, rows, cols, code, scale, zp, gs, code2 = spec.row(rec, out)
            table.add(src, dst, rows, cols, code, which, scale, zp, gs, code2)
            outs[i] = out
        table.launch(entry, *entry_args, _lib.stream_of(device))
        calls[group] = calls.get(group, 0) + 1

    # `recs` may be a generator: a call goes out as soon as its rows are there
    for i, rec in enumerate(recs):
        outs.append(None)
        key = spec.key(rec)
        if key is None:
            continue
        shape, dtype, device = spec.out_spec(rec)
        group = (dtype, device)
        rows = pending.setdefault(group, [])
        rows.append((i, rec, key, tuple(shape)))
        k = calls.get(group, 0)
        if len(rows) >= (_RAMP[k] if k < len(_RAMP) else _CHUNK_MODULES):
            flush(group)
    for group in list(pending):
        flush(group)
    return outs


def slab_outputs(shapes: List[Tuple[int, ...]], dtype: torch.dtype, device) -> List[torch.Tensor]:
    """one uninitialised tensor per entry of `shapes`.  Tensors of one shape are slices of a
    common allocation (up to 1 GiB each) where every slice stays 256-byte aligned: hundreds
    of outputs then cost a few allocator calls.  Slices of one allocation are freed together."""
    out: List[torch.Tensor] = [None] * len(shapes)
    by_shape: Dict[Tuple[int, ...], List[int]] = {}
    for i, shape in enumerate(shapes):
        by_shape.setdefault(shape, []).append(i)
    itemsize = torch.empty((), dtype=dtype).element_size()
    for shape, where in by_shape.items():
        nbytes = itemsize
        for d in shape:
            nbytes *= d
        per_slab = min(len(where), max(1, _SLAB_BYTES // max(nbytes, 1)))
        if nbytes == 0 or nbytes % _ALIGN or per_slab == 1:
            for i in where:
                out[i] = torch.empty(shape, dtype=dtype, device=device)
            continue
        for at in range(0, len(where), per_slab):
            part = where[at:at + per_slab]
            for i, t in zip(part, torch.empty((len(part),) + shape, dtype=dtype, device=device).unbind(0)):
                out[i] = t
    return out
