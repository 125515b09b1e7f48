"""`sparse-bitmask`: non-zero values + packed bitmask + row offsets.

Reference: compressors/sparse_compressors/sparse_bitmask.py (BitmaskCompressor
:35-57, BitmaskTensor :60-128, bitmask_compress :131-149, bitmask_decompress
:152-169).  The size of `compressed` depends on the data, so compression is two
kernels around one 8-byte read-back of the non-zero count.
"""
from typing import Dict, List, Tuple, Union

import torch
from torch import Tensor

from compressed_tensors_amd import _lib
from compressed_tensors_amd.compressors.base import BaseCompressor, to_gpu
from compressed_tensors_amd.compressors.sparse_base import BaseSparseCompressor
from compressed_tensors_amd.config import CompressionFormat
from compressed_tensors_amd.utils.helpers import merge_names

__all__ = ["BitmaskCompressor", "BitmaskTensor", "bitmask_compress", "bitmask_compress_many",
           "bitmask_decompress"]

_MANY = 64                 # weights per wait for the GPU in BitmaskCompressor.compress
_MOVED_BYTES = 1 << 30     # ... and of host weights copied to the GPU for it
_FLOAT_LIKE = (torch.float32, torch.float16, torch.bfloat16, torch.float8_e4m3fn)
_INT_LIKE = (torch.int8, torch.uint8, torch.int16, torch.int32, torch.bool)


def _elem(dtype: torch.dtype) -> Tuple[int, int]:
    if dtype in _FLOAT_LIKE:
        return torch.finfo(dtype).bits // 8, 1
    if dtype in _INT_LIKE:
        return (1 if dtype == torch.bool else torch.iinfo(dtype).bits // 8), 0
    raise NotImplementedError(f"bitmask compression of dtype {dtype} is not supported")


def bitmask_compress(tensor: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
    """dense [R, C] -> (values [nnz], bitmask uint8 [R, ceil(C/8)], row_offsets int64 [R])"""
    x = to_gpu(tensor).contiguous()
    if x.ndim < 1:
        raise ValueError("cannot compress a 0-d tensor")
    esize, is_float = _elem(x.dtype)
    cols = x.shape[-1]
    rows = x.numel() // cols if cols else 0
    lead = tuple(x.shape[:-1])
    dev = x.device
    lib = _lib.load()
    bitmask = torch.empty(lead + ((cols + 7) // 8,), dtype=torch.uint8, device=dev)
    # row_offsets follows cumsum over dim 0 of the per-row counts; for the 2-D
    # tensors this format is used with that is one offset per row
    if x.ndim != 2:
        raise NotImplementedError("bitmask compression expects a 2-D tensor")
    row_offsets = torch.empty((rows,), dtype=torch.int64, device=dev)
    total = torch.empty((1,), dtype=torch.int64, device=dev)
    tmp = torch.empty((lib.ctmi_bitmask_tmp_bytes(rows, cols),), dtype=torch.uint8, device=dev)
    stream = _lib.stream_of(dev)
    _lib.check(
        lib.ctmi_bitmask_count(
            x.data_ptr(), esize, is_float, bitmask.data_ptr(), row_offsets.data_ptr(),
            total.data_ptr(), tmp.data_ptr(), rows, cols, stream,
        )
    )
    nnz = int(total.item())  # the one unavoidable host read: sizes the output
    values = torch.empty((nnz,), dtype=x.dtype, device=dev)
    _lib.check(
        lib.ctmi_bitmask_compact(
            x.data_ptr(), esize, bitmask.data_ptr(), row_offsets.data_ptr(), values.data_ptr(),
            rows, cols, stream,
        )
    )
    return values, bitmask, row_offsets


def bitmask_compress_many(tensors: List[Tensor]) -> List[Tuple[Tensor, Tensor, Tensor]]:
    """bitmask_compress for a list of 2-D tensors with one host read for all of them: the
    mask-and-count passes of every tensor are enqueued first, the totals come back together,
    then the compaction passes follow (a state dict of N weights waits for the GPU once, not
    N times)."""
    lib = _lib.load()
    xs = [to_gpu(t).contiguous() for t in tensors]
    for x in xs:
        if x.ndim != 2:
            raise NotImplementedError("bitmask compression expects a 2-D tensor")
    out: List = [None] * len(xs)
    by_device: Dict[torch.device, List[int]] = {}
    for i, x in enumerate(xs):
        by_device.setdefault(x.device, []).append(i)
    for dev, idx in by_device.items():
        stream = _lib.stream_of(dev)
        totals = torch.empty((len(idx),), dtype=torch.int64, device=dev)
        held = []
        for k, i in enumerate(idx):
            x = xs[i]
            esize, is_float = _elem(x.dtype)
            rows, cols = x.shape
            bitmask = torch.empty((rows, (cols + 7) // 8), dtype=torch.uint8, device=dev)
            row_offsets = torch.empty((rows,), dtype=torch.int64, device=dev)
            tmp = torch.empty((lib.ctmi_bitmask_tmp_bytes(rows, cols),), dtype=torch.uint8, device=dev)
            _lib.check(lib.ctmi_bitmask_count(
                x.data_ptr(), esize, is_float, bitmask.data_ptr(), row_offsets.data_ptr(),
                totals.data_ptr() + 8 * k, tmp.data_ptr(), rows, cols, stream))
            held.append((bitmask, row_offsets, tmp, esize))
        counts = totals.tolist()  # the one host read: sizes the outputs
        for k, i in enumerate(idx):
            x = xs[i]
            bitmask, row_offsets, _, esize = held[k]
            values = torch.empty((counts[k],), dtype=x.dtype, device=dev)
            _lib.check(lib.ctmi_bitmask_compact(
                x.data_ptr(), esize, bitmask.data_ptr(), row_offsets.data_ptr(), values.data_ptr(),
                x.shape[0], x.shape[1], stream))
            out[i] = (values, bitmask, row_offsets)
    return out


def _scatter(values: Tensor, bitmasks: Tensor, row_offsets, shape, two_four: bool = False) -> Tensor:
    values = to_gpu(values).contiguous().reshape(-1)
    bitmasks = to_gpu(bitmasks).contiguous()
    shape = [int(d) for d in shape]
    cols = shape[-1]
    rows = 1
    for d in shape[:-1]:
        rows *= d
    esize, _ = _elem(values.dtype)
    dev = values.device
    lib = _lib.load()
    if bitmasks.numel() != rows * ((cols + 7) // 8):
        raise ValueError(f"bitmask of {bitmasks.numel()} bytes does not describe shape {shape}")
    out = torch.empty(shape, dtype=values.dtype, device=dev)
    tmp_bytes = (lib.ctmi_sparse24_tmp_bytes(rows, cols, esize) if two_four
                 else lib.ctmi_bitmask_tmp_bytes(rows, cols))
    tmp = torch.empty((tmp_bytes,), dtype=torch.uint8, device=dev)
    ro_ptr = None
    if row_offsets is not None:
        row_offsets = to_gpu(row_offsets).to(torch.int64).contiguous()
        ro_ptr = row_offsets.data_ptr()
    if two_four:
        rc = lib.ctmi_sparse24_decompress(
            values.data_ptr(), values.numel(), esize, bitmasks.data_ptr(), out.data_ptr(),
            tmp.data_ptr(), rows, cols, _lib.stream_of(dev),
        )
    else:
        rc = lib.ctmi_bitmask_decompress(
            values.data_ptr(), values.numel(), esize, bitmasks.data_ptr(), ro_ptr, out.data_ptr(),
            tmp.data_ptr(), rows, cols, _lib.stream_of(dev),
        )
    _lib.check(rc)
    return out


def bitmask_decompress(values: Tensor, bitmasks: Tensor, original_shape: torch.Size) -> Tensor:
    """zero-filled `original_shape` with `values` scattered to the set bits (row-major)"""
    return _scatter(values, bitmasks, None, original_shape)


class BitmaskTensor:
    """shape / compressed / bitmask / row_offsets of one compressed tensor"""

    def __init__(self, shape: Union[torch.Size, List], compressed: Tensor, bitmask: Tensor,
                 row_offsets: Tensor):
        self.shape = [int(d) for d in (shape.flatten().tolist() if isinstance(shape, Tensor) else shape)]
        self.compressed = compressed
        self.bitmask = bitmask
        self.row_offsets = row_offsets

    @staticmethod
    def from_dense(tensor: Tensor) -> "BitmaskTensor":
        compressed, bitmask, row_offsets = bitmask_compress(tensor)
        return BitmaskTensor(tensor.shape, compressed, bitmask, row_offsets)

    def decompress(self) -> Tensor:
        # like the reference, decompression derives positions from the bitmask alone
        return _scatter(self.compressed, self.bitmask, None, self.shape)

    def curr_memory_size_bytes(self) -> int:
        return sum(t.element_size() * t.nelement()
                   for t in (self.compressed, self.bitmask, self.row_offsets))

    def dict(self, name_prefix: str, device=None) -> Dict[str, Tensor]:
        def mv(t):
            return t if device is None else t.to(device)

        return {
            merge_names(name_prefix, "shape"): mv(torch.tensor(self.shape)),
            merge_names(name_prefix, "compressed"): mv(self.compressed),
            merge_names(name_prefix, "bitmask"): mv(self.bitmask),
            merge_names(name_prefix, "row_offsets"): mv(self.row_offsets),
        }

    def __repr__(self) -> str:
        return f"BitmaskTensor(shape={self.shape}, compressed=True)"


@BaseCompressor.register(name=CompressionFormat.sparse_bitmask.value)
class BitmaskCompressor(BaseSparseCompressor):
    @property
    def compression_param_names(self) -> Tuple[str]:
        return ("shape", "compressed", "bitmask", "row_offsets")

    def compress_weight(self, name, value):
        return BitmaskTensor.from_dense(value).dict(name_prefix=name, device=self.output_device)

    def compress(self, model_state, compression_targets=None, show_progress: bool = False):
        """BaseSparseCompressor.compress (sparse_compressors/base.py:66-112) with one wait for
        the GPU for all weights (bitmask_compress_many): same keys, order and values as the
        loop over compress_weight"""
        names = [n for n, v in model_state.items()
                 if self.should_compress(n, compression_targets) and isinstance(v, Tensor) and v.ndim == 2]
        if len(names) < 2:
            return super().compress(model_state, compression_targets, show_progress)
        # a batch at a time: weights that have to be copied to the GPU first stay there for
        # the length of their batch only
        packed, batch, moved = {}, [], 0
        for n in names + [None]:
            if n is not None:
                batch.append(n)
                v = model_state[n]
                moved += 0 if v.device.type == "cuda" else v.numel() * v.element_size()
            if batch and (n is None or len(batch) >= _MANY or moved >= _MOVED_BYTES):
                packed.update(zip(batch, bitmask_compress_many([model_state[b] for b in batch])))
                batch, moved = [], 0
        out: Dict[str, Tensor] = {}
        for name, value in model_state.items():
            if name in packed:
                values, bitmask, row_offsets = packed[name]
                prefix = name[: -len(".weight")]
                out.update(BitmaskTensor(value.shape, values, bitmask, row_offsets).dict(
                    name_prefix=prefix, device=self.output_device))
            elif self.should_compress(name, compression_targets):
                out.update(self.compress_weight(name[: -len(".weight")], value))
            else:
                out[name] = value
        return out

    def decompress_weight(self, weight_data):
        return BitmaskTensor(**weight_data).decompress()
