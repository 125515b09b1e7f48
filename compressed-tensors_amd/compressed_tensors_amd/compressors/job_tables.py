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

__all__ = ["WeightJobTable", "slab_outputs"]

_JOB = np.dtype(_lib.WeightJob)
_QP = np.dtype(_lib.QParams)
assert _JOB.itemsize == ctypes.sizeof(_lib.WeightJob) and _QP.itemsize == ctypes.sizeof(_lib.QParams)
_JOB_PTR = ctypes.POINTER(_lib.WeightJob)

_SLAB_BYTES = 1 << 30   # outputs of one shape share an allocation up to this size
_ALIGN = 256            # ... if each of them keeps this alignment inside it


class WeightJobTable:
    """Rows are added with `add`; `launch` writes them into a `ctmi_weight_job` array and
    hands it to a many-weight entry point.  `add_template` registers the part of a job's
    qparams that holds no scale or zero-point address (as `build_qparams` made it for one
    weight of the combination; its other addresses must be NULL)."""

    def __init__(self):
        self._templates: List[np.ndarray] = []
        self._template_of: Dict[Tuple, int] = {}
        self.clear()

    def clear(self):
        """drop the rows added since the last launch"""
        self.src, self.dst, self.rows, self.cols, self.dense_dtype = [], [], [], [], []
        self.scale, self.zero_point, self.which = [], [], []

    @property
    def n_templates(self) -> int:
        return len(self._templates)

    def template(self, key) -> int:
        """index of the template registered under `key`, or -1"""
        return self._template_of.get(key, -1)

    def add_template(self, key, plan) -> int:
        qp = np.frombuffer(bytes(plan.qp), dtype=_QP).copy()
        if int(qp["col_group"][0]) or int(qp["global_scale"][0]):
            raise ValueError("a template cannot hold the address of a column-group table or a global scale")
        qp["scale"] = 0
        qp["zero_point"] = 0
        self._templates.append(qp)
        self._stacked = np.concatenate(self._templates)
        self._template_of[key] = len(self._templates) - 1
        return len(self._templates) - 1

    def add(self, src: int, dst: int, rows: int, cols: int, dense_dtype: int, which: int,
            scale: int, zero_point: int = 0) -> None:
        self.src.append(src)
        self.dst.append(dst)
        self.rows.append(rows)
        self.cols.append(cols)
        self.dense_dtype.append(dense_dtype)
        self.which.append(which)
        self.scale.append(scale)
        self.zero_point.append(zero_point)

    def __len__(self):
        return len(self.src)

    def launch(self, entry, stream: int) -> None:
        """one call of `entry(jobs, n, stream)` for the rows added since the last launch"""
        n = len(self.src)
        if n == 0:
            return
        tab = np.zeros(n, _JOB)
        tab["src"] = self.src
        tab["dst"] = self.dst
        tab["rows"] = self.rows
        tab["cols"] = self.cols
        tab["dense_dtype"] = self.dense_dtype
        qp = self._stacked[self.which]
        qp["scale"] = self.scale
        qp["zero_point"] = self.zero_point
        tab["qp"] = qp
        self.clear()
        # the entry points read the table before they return: it need not outlive the call
        _lib.check(entry(ctypes.cast(tab.ctypes.data, _JOB_PTR), n, stream))


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
