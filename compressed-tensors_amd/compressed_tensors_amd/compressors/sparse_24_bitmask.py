"""`sparse-24-bitmask`: the two survivors of every group of four + packed bitmask.

Reference: compressors/sparse_compressors/sparse_24_bitmask.py
(Sparse24BitMaskCompressor :37-67, Sparse24BitMaskTensor :70-159,
sparse24_bitmask_compress :162-203, sparse24_bitmask_decompress :206-224,
get_24_bytemasks :227-260).
"""
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple, Union

import torch
from torch import Tensor

from compressed_tensors_amd import _lib
from compressed_tensors_amd.compressors.base import BaseCompressor, to_gpu
from compressed_tensors_amd.compressors.sparse_base import BaseSparseCompressor
from compressed_tensors_amd.compressors.sparse_bitmask import _scatter
from compressed_tensors_amd.config import CompressionFormat, SparsityStructure
from compressed_tensors_amd.utils.helpers import merge_names

__all__ = [
    "Sparse24BitMaskCompressor",
    "Sparse24BitMaskTensor",
    "sparse24_bitmask_compress",
    "sparse24_bitmask_decompress",
    "sparse24_bitmask_compress_many",
    "sparse24_bitmask_decompress_many",
    "quantize_sparse24_compress",
    "quantize_sparse24_compress_many",
    "sparse24_decompress_dequantize",
    "sparse24_decompress_dequantize_many",
    "get_24_bytemasks",
]

_RANKABLE = (torch.float32, torch.float16, torch.bfloat16, torch.float8_e4m3fn, torch.int8)


def _check_dtype(dtype: torch.dtype) -> None:
    if dtype not in _RANKABLE:
        raise NotImplementedError(f"2:4 masks of dtype {dtype} are not supported")


def get_24_bytemasks(tensor: Tensor) -> Tensor:
    """bool mask keeping, in every run of four elements, the two that
    `abs().topk(2)` keeps (float8 tensors are ranked through their int8 view)."""
    x = to_gpu(tensor).contiguous()
    _check_dtype(x.dtype)
    if x.numel() % 4 != 0:
        raise ValueError("Tensor size must be a multiple of 4 for TWO_FOUR sparsity")
    mask = torch.empty(x.shape, dtype=torch.bool, device=x.device)
    _lib.check(
        _lib.load().ctmi_get_24_bytemasks(
            x.data_ptr(), _lib.dtype_code(x.dtype), mask.data_ptr(), x.numel(),
            _lib.stream_of(x.device),
        )
    )
    return mask


def sparse24_bitmask_compress(
    tensor: Tensor,
    sparsity_structure: Union[SparsityStructure, str] = SparsityStructure.TWO_FOUR,
) -> Tuple[Tensor, Tensor]:
    """dense [R, C] -> (values [R, C/2], bitmask uint8 [R, ceil(C/8)])"""
    assert len(tensor.shape) == 2, "Only 2D tensors are supported"
    assert (
        SparsityStructure(sparsity_structure) == SparsityStructure.TWO_FOUR
    ), "Only 2:4 sparsity is supported"
    rows, cols = tensor.shape
    if tensor.is_meta:
        return (
            torch.empty((rows, cols // 2), dtype=tensor.dtype, device="meta"),
            torch.empty((rows, (cols + 7) // 8), dtype=torch.uint8, device="meta"),
        )
    x = to_gpu(tensor).contiguous()
    _check_dtype(x.dtype)
    if x.numel() % 4 != 0:
        raise ValueError("Tensor size must be a multiple of 4 for TWO_FOUR sparsity")
    values = torch.empty((rows, cols // 2), dtype=x.dtype, device=x.device)
    bitmask = torch.empty((rows, (cols + 7) // 8), dtype=torch.uint8, device=x.device)
    _lib.check(
        _lib.load().ctmi_sparse24_compress(
            x.data_ptr(), _lib.dtype_code(x.dtype), values.data_ptr(), bitmask.data_ptr(), rows,
            cols, _lib.stream_of(x.device),
        )
    )
    return values, bitmask


def _streams(rows: int, cols: int, esize: int, decompress: bool) -> bool:
    """the shapes the multi-tensor entry points take: rows of whole bitmask bytes and a
    whole number of work items"""
    per = 16 if esize == 1 else 8
    return rows > 0 and cols > 0 and cols % 8 == 0 and (rows * cols) % per == 0


def sparse24_bitmask_compress_many(tensors: List[Tensor]) -> List[Tuple[Tensor, Tensor]]:
    """sparse24_bitmask_compress on several 2-D tensors: those of one dtype go to the GPU
    in one call (ctmi_sparse24_compress_many, 8 tensors per launch); shapes it does not
    take get a call of their own.  Same bits either way."""
    results: List[Optional[Tuple[Tensor, Tensor]]] = [None] * len(tensors)
    by_dtype: Dict[torch.dtype, List[int]] = {}
    xs: List[Optional[Tensor]] = [None] * len(tensors)
    for i, t in enumerate(tensors):
        if t.is_meta or t.ndim != 2 or t.dtype not in _RANKABLE or not _streams(
                t.shape[0], t.shape[1], t.element_size(), False):
            results[i] = sparse24_bitmask_compress(t)
            continue
        xs[i] = to_gpu(t).contiguous()
        by_dtype.setdefault(t.dtype, []).append(i)
    lib = _lib.load()
    for dtype, idx in by_dtype.items():
        dev = xs[idx[0]].device
        idx_here = [i for i in idx if xs[i].device == dev]
        for i in idx:
            if xs[i].device != dev:
                results[i] = sparse24_bitmask_compress(xs[i])
        jobs = (_lib.Sparse24Job * len(idx_here))()
        for job, i in zip(jobs, idx_here):
            x = xs[i]
            rows, cols = x.shape
            values = torch.empty((rows, cols // 2), dtype=dtype, device=dev)
            bitmask = torch.empty((rows, cols // 8), dtype=torch.uint8, device=dev)
            job.dense, job.values, job.bitmask = x.data_ptr(), values.data_ptr(), bitmask.data_ptr()
            job.nvalues, job.rows, job.cols = values.numel(), rows, cols
            results[i] = (values, bitmask)
        _lib.check(lib.ctmi_sparse24_compress_many(jobs, len(idx_here), _lib.dtype_code(dtype),
                                                   _lib.stream_of(dev)))
    return results


def sparse24_bitmask_decompress_many(items: List[Tuple[Tensor, Tensor, List[int]]]) -> List[Tensor]:
    """sparse24_bitmask_decompress on several (values, bitmask, shape) triples: those of one
    element size go to the GPU in one call (ctmi_sparse24_decompress_many)"""
    results: List[Optional[Tensor]] = [None] * len(items)
    groups: Dict[Tuple[torch.dtype, str], List[int]] = {}
    prepared = {}
    for i, (values, bitmask, shape) in enumerate(items):
        shape = [int(d) for d in (shape.flatten().tolist() if isinstance(shape, Tensor) else shape)]
        rows = 1
        for d in shape[:-1]:
            rows *= d
        cols = shape[-1] if shape else 0
        ok = (not values.is_meta and len(shape) >= 1 and _streams(rows, cols, values.element_size(), True)
              and values.numel() * 2 == rows * cols and bitmask.numel() * 8 == rows * cols
              and values.element_size() in (1, 2, 4))
        if not ok:
            results[i] = sparse24_bitmask_decompress(values, bitmask, shape)
            continue
        v, b = to_gpu(values).contiguous().reshape(-1), to_gpu(bitmask).contiguous()
        prepared[i] = (v, b, shape, rows, cols)
        groups.setdefault((v.dtype, str(v.device)), []).append(i)
    lib = _lib.load()
    for (dtype, _), idx in groups.items():
        dev = prepared[idx[0]][0].device
        jobs = (_lib.Sparse24Job * len(idx))()
        for job, i in zip(jobs, idx):
            v, b, shape, rows, cols = prepared[i]
            out = torch.empty(shape, dtype=dtype, device=dev)
            job.dense, job.values, job.bitmask = out.data_ptr(), v.data_ptr(), b.data_ptr()
            job.nvalues, job.rows, job.cols = v.numel(), rows, cols
            results[i] = out
        _lib.check(lib.ctmi_sparse24_decompress_many(jobs, len(idx), v.element_size(),
                                                     _lib.stream_of(dev)))
    return results


def quantize_sparse24_compress(weight: Tensor, scale: Tensor, quantization_args,
                               zero_point: Optional[Tensor] = None,
                               g_idx: Optional[Tensor] = None) -> Optional[Tuple[Tensor, Tensor]]:
    """quantize(weight, dtype=args.pytorch_dtype()) followed by sparse24_bitmask_compress of
    the codes, in one pass over the weight: (values [R, C/2] in the code dtype, bitmask).
    None when the layout has no fused kernel (the caller then takes the two steps)."""
    import ctypes

    from compressed_tensors_amd.quantization.forward import build_qparams
    from compressed_tensors_amd.quantization.helpers import can_quantize

    if g_idx is not None or weight.ndim != 2 or weight.is_meta or not can_quantize(weight, quantization_args):
        return None
    w, scale, zero_point = (to_gpu(t) for t in (weight, scale, zero_point))
    w = w.contiguous()
    rows, cols = w.shape
    if rows == 0 or cols == 0 or w.data_ptr() % (8 * w.element_size()):
        return None
    plan = build_qparams(w, scale, zero_point, quantization_args, None, None)
    lib = _lib.load()
    if not lib.ctmi_quantize_sparse24_compress_supported(_lib.dtype_code(w.dtype), rows, cols,
                                                         ctypes.byref(plan.qp)):
        return None
    values = torch.empty((rows, cols // 2), dtype=quantization_args.pytorch_dtype(), device=w.device)
    bitmask = torch.empty((rows, cols // 8), dtype=torch.uint8, device=w.device)
    _lib.check(
        lib.ctmi_quantize_sparse24_compress(
            w.data_ptr(), _lib.dtype_code(w.dtype), values.data_ptr(), bitmask.data_ptr(), rows, cols,
            ctypes.byref(plan.qp), _lib.stream_of(w.device),
        )
    )
    return values, bitmask


def sparse24_decompress_dequantize(values: Tensor, bitmask: Tensor, original_shape, scale: Tensor,
                                   zero_point: Optional[Tensor] = None,
                                   g_idx: Optional[Tensor] = None,
                                   quantization_args=None) -> Optional[Tensor]:
    """sparse24_bitmask_decompress of int8 / float8 codes followed by dequantize(codes,
    scale, zero_point) (dtype: the scale's), in one pass over the compressed weight.
    None when the layout has no fused kernel (the caller then takes the two steps)."""
    import ctypes

    from compressed_tensors_amd.quantization.forward import (
        _ShapeOnly, build_qparams, infer_dequant_args,
    )

    shape = [int(d) for d in (original_shape.flatten().tolist()
                              if isinstance(original_shape, Tensor) else original_shape)]
    if (g_idx is not None or len(shape) != 2 or values.is_meta
            or values.dtype not in (torch.int8, torch.float8_e4m3fn)
            or scale.dtype not in (torch.bfloat16, torch.float16, torch.float32)):
        return None
    rows, cols = shape
    values, bitmask, scale, zero_point = (to_gpu(t) for t in (values, bitmask, scale, zero_point))
    values, bitmask = values.contiguous(), bitmask.contiguous()
    if (rows == 0 or cols == 0 or cols % 8 or values.numel() * 2 != rows * cols
            or bitmask.numel() * 8 != rows * cols or values.data_ptr() % 4):
        return None
    codes = _ShapeOnly(shape, values.dtype)
    args = quantization_args if quantization_args is not None else infer_dequant_args(codes, scale)
    plan = build_qparams(codes, scale, zero_point, args, None, None)
    lib = _lib.load()
    vcode, ocode = _lib.dtype_code(values.dtype), _lib.dtype_code(scale.dtype)
    if not lib.ctmi_sparse24_decompress_dequantize_supported(vcode, ocode, rows, cols,
                                                             ctypes.byref(plan.qp)):
        return None
    out = torch.empty((rows, cols), dtype=scale.dtype, device=values.device)
    tmp = torch.empty(lib.ctmi_sparse24_dequantize_tmp_bytes(rows, cols), dtype=torch.uint8,
                      device=values.device)
    _lib.check(
        lib.ctmi_sparse24_decompress_dequantize(
            values.data_ptr(), values.numel(), vcode, bitmask.data_ptr(), out.data_ptr(), ocode,
            tmp.data_ptr(), rows, cols, ctypes.byref(plan.qp), _lib.stream_of(values.device),
        )
    )
    return out


# What decides the qparams of a stacked weight besides addresses -> (the qparams as bytes, does
# the fused kernel take the layout?): a model has a handful of such combinations.
_stacked_compress_plans: Dict[Tuple, Tuple[bytes, bool]] = {}
_stacked_decompress_plans: Dict[Tuple, Tuple[bytes, bool]] = {}
_FLOATS = (torch.bfloat16, torch.float16, torch.float32)


def _stacked_call(entry, rows, device) -> None:
    """one many-weight call for `rows` = (dense, values, bitmask, n_rows, n_cols, dense code,
    values code, qparams bytes, scale, zero_point) tuples: the job table written by columns"""
    import ctypes

    import numpy as np

    job_t, qp_t = np.dtype(_lib.Stacked24Job), np.dtype(_lib.QParams)
    tab = np.zeros(len(rows), job_t)
    cols = list(zip(*rows))
    for name, col in zip(("dense", "values", "bitmask", "rows", "cols", "dense_dtype", "values_dtype"), cols):
        tab[name] = col
    qp = np.frombuffer(b"".join(cols[7]), dtype=qp_t).copy()
    qp["scale"] = cols[8]
    qp["zero_point"] = cols[9]
    tab["qp"] = qp
    _lib.check(entry(ctypes.cast(tab.ctypes.data, ctypes.POINTER(_lib.Stacked24Job)), len(rows),
                     _lib.stream_of(device)))


_STACKED_CALL = 32  # weights per call (4 launches of 8): the GPU starts while later rows are written


def quantize_sparse24_compress_many(recs) -> List[Optional[Tuple[Tensor, Tensor]]]:
    """quantize_sparse24_compress for (weight, scale, zero_point, args) records whose tensors are
    on the GPU already, through ctmi_quantize_sparse24_compress_many (8 weights per launch):
    the qparams of a (shape, dtype, scheme) combination are derived once, outputs of one shape
    share allocations.  None for records this does not take."""
    import ctypes

    from compressed_tensors_amd.compressors.job_tables import args_key, on_gpu, slab_outputs
    from compressed_tensors_amd.quantization.forward import build_qparams

    lib = _lib.load()
    outs: List[Optional[Tuple[Tensor, Tensor]]] = [None] * len(recs)
    groups: Dict[Tuple, List] = {}
    for i, (w, scale, zp, args) in enumerate(recs):
        if (not on_gpu(w) or w.ndim != 2 or w.numel() == 0 or w.dtype not in _FLOATS
                or w.data_ptr() % (8 * w.element_size()) or not on_gpu(scale, w.device)
                or scale.dtype not in _FLOATS or scale.ndim == 0 or args.num_bits > 8
                or (zp is not None and not on_gpu(zp, w.device))):
            continue
        key = (w.shape, w.dtype, scale.shape, scale.dtype, None if zp is None else zp.dtype, args_key(args))
        plan = _stacked_compress_plans.get(key)
        if plan is None:
            if len(_stacked_compress_plans) > 1024:
                _stacked_compress_plans.clear()
            qplan = build_qparams(w, scale, zp, args, None, None)
            ok = bool(lib.ctmi_quantize_sparse24_compress_supported(
                _lib.dtype_code(w.dtype), w.shape[0], w.shape[1], ctypes.byref(qplan.qp)))
            plan = _stacked_compress_plans[key] = (bytes(qplan.qp), ok)
        if plan[1]:
            groups.setdefault((args.pytorch_dtype(), w.device), []).append((i, plan[0]))
    for (code_dtype, device), items in groups.items():
        vcode = _lib.dtype_code(code_dtype)
        for at in range(0, len(items), _STACKED_CALL):
            part = items[at:at + _STACKED_CALL]
            values = slab_outputs([(recs[i][0].shape[0], recs[i][0].shape[1] // 2) for i, _ in part], code_dtype, device)
            bitmasks = slab_outputs([(recs[i][0].shape[0], recs[i][0].shape[1] // 8) for i, _ in part], torch.uint8, device)
            rows = []
            for (i, raw), v, b in zip(part, values, bitmasks):
                w, scale, zp, _ = recs[i]
                rows.append((w.data_ptr(), v.data_ptr(), b.data_ptr(), w.shape[0], w.shape[1],
                             _lib.dtype_code(w.dtype), vcode, raw, scale.data_ptr(),
                             0 if zp is None else zp.data_ptr()))
                outs[i] = (v, b)
            _stacked_call(lib.ctmi_quantize_sparse24_compress_many, rows, device)
    return outs


def sparse24_decompress_dequantize_many(recs) -> List[Optional[Tensor]]:
    """sparse24_decompress_dequantize for (values, bitmask, shape, scale, zero_point) records
    whose tensors are on the GPU already (shape: a pair of ints), through
    ctmi_sparse24_decompress_dequantize_many; None for records this does not take"""
    import ctypes

    from compressed_tensors_amd.compressors.job_tables import on_gpu, slab_outputs
    from compressed_tensors_amd.quantization.forward import _ShapeOnly, build_qparams, infer_dequant_args

    lib = _lib.load()
    outs: List[Optional[Tensor]] = [None] * len(recs)
    groups: Dict[Tuple, List] = {}
    for i, (values, bitmask, shape, scale, zp) in enumerate(recs):
        if (len(shape) != 2 or not on_gpu(values) or values.dtype not in (torch.int8, torch.float8_e4m3fn)
                or not on_gpu(bitmask, values.device) or not on_gpu(scale, values.device)
                or scale.dtype not in _FLOATS or (zp is not None and not on_gpu(zp, values.device))):
            continue
        rows, cols = shape
        if (rows == 0 or cols == 0 or cols % 8 or values.numel() * 2 != rows * cols
                or bitmask.numel() * 8 != rows * cols or values.data_ptr() % 4):
            continue
        key = (rows, cols, values.dtype, scale.shape, scale.dtype, None if zp is None else zp.dtype)
        plan = _stacked_decompress_plans.get(key)
        if plan is None:
            if len(_stacked_decompress_plans) > 1024:
                _stacked_decompress_plans.clear()
            codes = _ShapeOnly((rows, cols), values.dtype)
            qplan = build_qparams(codes, scale, zp, infer_dequant_args(codes, scale), None, None)
            ok = bool(lib.ctmi_sparse24_decompress_dequantize_supported(
                _lib.dtype_code(values.dtype), _lib.dtype_code(scale.dtype), rows, cols, ctypes.byref(qplan.qp)))
            plan = _stacked_decompress_plans[key] = (bytes(qplan.qp), ok)
        if plan[1]:
            groups.setdefault((scale.dtype, values.device), []).append((i, plan[0]))
    for (dtype, device), items in groups.items():
        ocode = _lib.dtype_code(dtype)
        for at in range(0, len(items), _STACKED_CALL):
            part = items[at:at + _STACKED_CALL]
            dense = slab_outputs([tuple(recs[i][2]) for i, _ in part], dtype, device)
            rows = []
            for (i, raw), out in zip(part, dense):
                values, bitmask, shape, scale, zp = recs[i]
                rows.append((out.data_ptr(), values.data_ptr(), bitmask.data_ptr(), shape[0], shape[1],
                             ocode, _lib.dtype_code(values.dtype), raw, scale.data_ptr(),
                             0 if zp is None else zp.data_ptr()))
                outs[i] = out
            _stacked_call(lib.ctmi_sparse24_decompress_dequantize_many, rows, device)
    return outs


def sparse24_bitmask_decompress(
    values: Tensor, bitmasks: Tensor, original_shape: torch.Size
) -> Tensor:
    return _scatter(values, bitmasks, None, original_shape, two_four=True)


@dataclass
class Sparse24BitMaskTensor:
    shape: List[int]
    compressed: Tensor
    bitmask: Tensor

    @staticmethod
    def from_dense(
        tensor: Tensor,
        sparsity_structure: Union[SparsityStructure, str] = SparsityStructure.TWO_FOUR,
    ) -> "Sparse24BitMaskTensor":
        compressed, bitmask = sparse24_bitmask_compress(tensor, sparsity_structure)
        return Sparse24BitMaskTensor(shape=list(tensor.shape), compressed=compressed,
                                     bitmask=bitmask)

    @staticmethod
    def from_compressed_data(
        shape: Union[List[int], Tensor], compressed: Tensor, bitmask: Tensor
    ) -> "Sparse24BitMaskTensor":
        if isinstance(shape, Tensor):
            shape = shape.flatten().tolist()
        return Sparse24BitMaskTensor(shape=[int(d) for d in shape], compressed=compressed,
                                     bitmask=bitmask)

    def decompress(self) -> Tensor:
        return sparse24_bitmask_decompress(self.compressed, self.bitmask, self.shape)

    def curr_memory_size_bytes(self) -> int:
        return sum(t.element_size() * t.nelement() for t in (self.compressed, self.bitmask))

    def dict(self, name_prefix: str, device=None) -> Dict[str, Tensor]:
        if name_prefix.endswith(".weight"):
            name_prefix = name_prefix[: -len(".weight")]

        def mv(t):
            return t if device is None else t.to(device)

        return {
            merge_names(name_prefix, "shape"): mv(torch.tensor(self.shape).reshape(-1, 1)),
            merge_names(name_prefix, "compressed"): mv(self.compressed),
            merge_names(name_prefix, "bitmask"): mv(self.bitmask),
        }

    def __repr__(self) -> str:
        return f"BitMaskTensor(shape={self.shape}, compressed=True)"


@BaseCompressor.register(name=CompressionFormat.sparse_24_bitmask.value)
class Sparse24BitMaskCompressor(BaseSparseCompressor):
    @property
    def compression_param_names(self) -> Tuple[str]:
        return ("shape", "compressed", "bitmask")

    def compress_weight(self, name, value):
        structure = getattr(self.config, "sparsity_structure", SparsityStructure.TWO_FOUR.value)
        tensor = Sparse24BitMaskTensor.from_dense(value, structure)
        return tensor.dict(name_prefix=name,
                           device="meta" if value.is_meta else self.output_device)

    def decompress_weight(self, weight_data):
        return Sparse24BitMaskTensor.from_compressed_data(**weight_data).decompress()

    # the whole state dict in a few calls: the weights of one dtype share launches
    def compress(self, model_state, compression_targets=None, show_progress: bool = False):
        names = [n for n in model_state if self.should_compress(n, compression_targets)]
        structure = getattr(self.config, "sparsity_structure", SparsityStructure.TWO_FOUR.value)
        assert SparsityStructure(structure) == SparsityStructure.TWO_FOUR, "Only 2:4 sparsity is supported"
        for n in names:
            assert len(model_state[n].shape) == 2, "Only 2D tensors are supported"
        compressed = dict(zip(names, sparse24_bitmask_compress_many([model_state[n] for n in names])))
        out: Dict[str, Tensor] = {}
        for name, value in model_state.items():
            if name not in compressed:
                out[name] = value
                continue
            values, bitmask = compressed[name]
            tensor = Sparse24BitMaskTensor(shape=list(value.shape), compressed=values, bitmask=bitmask)
            out.update(tensor.dict(name_prefix=name,
                                   device="meta" if value.is_meta else self.output_device))
        return out

    def decompress_from_state_dict(self, state_dict):
        from compressed_tensors_amd.utils.helpers import nest_state_dict

        nested, ignored = nest_state_dict(state_dict, self.compression_param_names,
                                          return_unmatched_params=True)
        paths = list(nested)
        dense = sparse24_bitmask_decompress_many(
            [(nested[p]["compressed"], nested[p]["bitmask"], nested[p]["shape"]) for p in paths])
        for path, weight in zip(paths, dense):
            yield merge_names(path, "weight"), weight
        for name, value in ignored.items():
            yield name, value
