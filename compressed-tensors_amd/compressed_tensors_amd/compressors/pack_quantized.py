"""`pack-quantized`: integer weights packed 32/num_bits to an int32.

Reference: compressors/quantized_compressors/pack_quantized.py
(PackedQuantizationCompressor :33-183, pack_to_int32 :186-246,
unpack_from_int32 :249-309).  compress_weight / decompress_weight run as one
fused kernel each (quantize+pack, unpack+dequantize); the free functions pack
and unpack int8 tensors on their own.
"""
import ctypes
import math
from typing import Dict, Optional, Tuple

import torch
from torch import Tensor

from compressed_tensors_amd import _lib
from compressed_tensors_amd.compressors.base import BaseCompressor, to_gpu
from compressed_tensors_amd.compressors.job_tables import (
    FLOAT_DTYPES, args_key, on_gpu, run_table,
)
from compressed_tensors_amd.compressors.quantized_base import (
    BaseQuantizationCompressor, LazyDenseOutputs,
)
from compressed_tensors_amd.config import CompressionFormat
from compressed_tensors_amd.quantization.forward import (
    _ShapeOnly,
    _column_groups,
    build_qparams,
    infer_dequant_args,
)
from compressed_tensors_amd.quantization.helpers import can_quantize
from compressed_tensors_amd.quantization.quant_args import QuantizationArgs, QuantizationStrategy

__all__ = ["PackedQuantizationCompressor", "PackedWeightBatch", "ObservedWeightBatch",
           "pack_to_int32", "unpack_from_int32"]

_PACKABLE = (QuantizationStrategy.GROUP.value, QuantizationStrategy.CHANNEL.value)
_CHUNK = 32  # weights per multi-weight call of the state-dict paths (4 launches of 8)


def pack_to_int32(value: Tensor, num_bits: int, packed_dim: int = 1) -> Tensor:
    """int8 [R, C] -> int32 [R, ceil(C/pf)] (or [ceil(R/pf), C] for packed_dim=0)."""
    if value.dtype is not torch.int8:
        raise ValueError("Tensor must be quantized to torch.int8 before packing")
    if num_bits > 8:
        raise ValueError("Packing is only supported for less than 8 bits")
    if num_bits < 1:
        raise ValueError(f"num_bits must be at least 1, got {num_bits}")
    if value.ndim != 2:
        raise ValueError(f"expected a 2-D tensor, got shape {tuple(value.shape)}")
    value = to_gpu(value).contiguous()
    rows, cols = value.shape
    pf = 32 // num_bits
    shape = (rows, math.ceil(cols / pf)) if packed_dim == 1 else (math.ceil(rows / pf), cols)
    out = torch.empty(shape, dtype=torch.int32, device=value.device)
    _lib.check(
        _lib.load().ctmi_pack_to_int32(
            value.data_ptr(), out.data_ptr(), rows, cols, num_bits, packed_dim,
            _lib.stream_of(value.device),
        )
    )
    return out


def unpack_from_int32(
    value: Tensor, num_bits: int, shape: torch.Size, packed_dim: int = 1
) -> Tensor:
    """inverse of pack_to_int32; `shape` is the unpacked shape (padding is cut off)."""
    if value.dtype is not torch.int32:
        raise ValueError(f"Expected {torch.int32} but got {value.dtype}, Aborting unpack.")
    if num_bits > 8:
        raise ValueError("Unpacking is only supported for less than 8 bits")
    value = to_gpu(value)
    pf = 32 // num_bits
    if packed_dim == 1:
        rows = value.shape[0]
        cols = min(int(shape[1]), value.shape[1] * pf)
        need = math.ceil(cols / pf)
        if value.shape[1] != need:
            value = value[:, :need]
    else:
        cols = value.shape[1]
        rows = min(int(shape[0]), value.shape[0] * pf)
        need = math.ceil(rows / pf)
        if value.shape[0] != need:
            value = value[:need, :]
    value = value.contiguous()
    out = torch.empty((rows, cols), dtype=torch.int8, device=value.device)
    _lib.check(
        _lib.load().ctmi_unpack_from_int32(
            value.data_ptr(), out.data_ptr(), rows, cols, num_bits, packed_dim,
            _lib.stream_of(value.device),
        )
    )
    return out


@BaseCompressor.register(name=CompressionFormat.pack_quantized.value)
class PackedQuantizationCompressor(BaseQuantizationCompressor):
    packs_zero_points = True

    @property
    def compression_param_names(self) -> Tuple[str]:
        return (
            "weight_packed",
            "weight_scale",
            "weight_zero_point",
            "weight_g_idx",
            "weight_shape",
        )

    def compression_param_info(
        self, weight_shape: torch.Size, quantization_args: Optional[QuantizationArgs] = None
    ) -> Dict[str, Tuple[torch.Size, torch.dtype]]:
        pf = 32 // quantization_args.num_bits
        info = {
            "weight_packed": (
                torch.Size((weight_shape[0], math.ceil(weight_shape[1] / pf))),
                torch.int32,
            ),
            "weight_shape": (torch.Size((2,)), torch.int32),
        }
        if not quantization_args.symmetric and quantization_args.strategy in _PACKABLE:
            zp_factor = (
                quantization_args.group_size
                if quantization_args.strategy == QuantizationStrategy.GROUP.value
                else weight_shape[-1]
            )
            info["weight_zero_point"] = (
                torch.Size((math.ceil(weight_shape[0] / pf), weight_shape[-1] // zp_factor)),
                torch.int32,
            )
        return info

    def compress_weight(
        self,
        weight: Tensor,
        scale: Tensor,
        quantization_args: QuantizationArgs,
        zero_point: Optional[Tensor] = None,
        g_idx: Optional[Tensor] = None,
        device: Optional[torch.device] = None,
        global_scale: Optional[Tensor] = None,
    ) -> Dict[str, Tensor]:
        if global_scale is not None:
            raise ValueError("global_scale is not supported for the PackQuantizationCompressor")
        args = quantization_args
        weight, scale, zero_point, g_idx = (to_gpu(t) for t in (weight, scale, zero_point, g_idx))

        if can_quantize(weight, args):
            if weight.ndim != 2:
                raise ValueError(f"expected a 2-D weight, got shape {tuple(weight.shape)}")
            plan = build_qparams(weight, scale, zero_point, args, g_idx, None)
            w = weight.contiguous()
            rows, cols = w.shape
            pf = 32 // max(1, min(args.num_bits, 32))
            packed = torch.empty(
                (rows, math.ceil(cols / max(pf, 1))), dtype=torch.int32, device=w.device
            )
            _lib.check(
                _lib.load().ctmi_pack_quantized_compress(
                    w.data_ptr(), _lib.dtype_code(w.dtype), packed.data_ptr(), rows, cols,
                    ctypes.byref(plan.qp), _lib.stream_of(w.device),
                )
            )
        else:
            packed = pack_to_int32(weight, args.num_bits)

        weight_shape = torch.tensor(weight.shape)
        if device is not None:
            packed = packed.to(device)
            weight_shape = weight_shape.to(device)
        out = {"weight_shape": weight_shape, "weight_packed": packed}
        if not args.symmetric and args.strategy in _PACKABLE:
            out["weight_zero_point"] = pack_to_int32(zero_point, args.num_bits, packed_dim=0)
        return out

    @staticmethod
    def one_pass_kernel(weight: Tensor, args: QuantizationArgs, g_idx: Optional[Tensor] = None):
        """which kernel compresses a weight without scales in one pass: "groups" (groups are
        runs of neighbouring lanes: column order, 8 ... 512 elements, a power of two; or one
        cell per row), "table" (the group of a column looked up or divided out: activation
        ordering, any group size) or None (the observer and the compressor run one after
        the other)"""
        if weight.ndim != 2 or args.type != "int" or not can_quantize(weight, args):
            return None
        rows, cols = weight.shape
        if args.strategy == QuantizationStrategy.GROUP.value:
            blk_cols = args.group_size
        elif args.strategy == QuantizationStrategy.CHANNEL.value:
            blk_cols, g_idx = cols, None
        else:
            return None
        if weight.data_ptr() % (8 * weight.element_size()) or weight.dtype not in _FLOAT_DTYPES:
            return None
        lib, code = _lib.load(), _lib.dtype_code(weight.dtype)
        if g_idx is None and lib.ctmi_observe_pack_quantized_supported(code, rows, cols, blk_cols, args.num_bits):
            return "groups"
        if g_idx is not None and g_idx.numel() >= 1 << 16:
            return None
        if lib.ctmi_observe_pack_quantized_gidx_supported(code, rows, cols, min(blk_cols, cols), args.num_bits):
            return "table"
        return None

    def observe_and_compress_weight(
        self, weight: Tensor, quantization_args: QuantizationArgs,
        device: Optional[torch.device] = None, g_idx: Optional[Tensor] = None,
    ) -> Dict[str, Tensor]:
        """One-shot (round-to-nearest) compression of a weight that has no scales yet:
        the min-max observer (tests/mock_observer.py:38-113), calculate_qparams
        (quantization/utils/helpers.py:67-146) and compress_weight
        (pack_quantized.py:88-146) in one pass over the weight for group and channel
        strategies, with or without activation ordering (`one_pass_kernel` says which kernel
        takes a weight); the other strategies (one scale per tensor, blocks) and rows beyond
        16384 elements run the observer and the compressor one after the other.  With g_idx
        the observer sees the columns in the order quantize groups them (sorted by g_idx,
        forward.py:286-303).  Returns compress_weight's dict plus "weight_scale" (and the
        packed "weight_zero_point" of an asymmetric scheme)."""
        args = quantization_args
        weight = to_gpu(weight)
        if weight.ndim != 2:
            raise ValueError(f"expected a 2-D weight, got shape {tuple(weight.shape)}")
        rows, cols = weight.shape
        if args.strategy == QuantizationStrategy.GROUP.value:
            blk_cols = args.group_size
        elif args.strategy == QuantizationStrategy.CHANNEL.value:
            blk_cols = cols
        else:
            blk_cols = 0
        lib = _lib.load()
        w = weight.contiguous()
        kernel = self.one_pass_kernel(w, args, g_idx)
        if kernel is None:
            from compressed_tensors_amd.quantization.helpers import observe_weight_qparams

            seen = weight
            if g_idx is not None and not bool((g_idx == -1).any()):
                seen = weight.index_select(1, torch.argsort(to_gpu(g_idx).long()))
            scale, zero_point = observe_weight_qparams(seen, args)
            out = self.compress_weight(weight, scale, args, zero_point=zero_point, g_idx=g_idx,
                                       device=device)
            out["weight_scale"] = scale if device is None else scale.to(device)
            return out
        n_cells = cols // min(blk_cols, cols)
        packed = torch.empty((rows, cols * args.num_bits // 32), dtype=torch.int32, device=w.device)
        scale = torch.empty((rows, n_cells), dtype=w.dtype, device=w.device)
        zero_point = None
        if not args.symmetric:
            zero_point = torch.empty((rows, n_cells), dtype=torch.int8, device=w.device)
        if kernel == "groups":
            _lib.check(
                lib.ctmi_observe_pack_quantized(
                    w.data_ptr(), _lib.dtype_code(w.dtype), rows, cols, blk_cols, args.num_bits,
                    int(args.symmetric), packed.data_ptr(), scale.data_ptr(), _lib.ptr(zero_point),
                    _lib.stream_of(w.device),
                )
            )
        else:
            # groups that are no runs of neighbouring lanes: the group of every column from a
            # table (activation ordering) or by division (any group size)
            col_group = None
            if g_idx is not None and args.strategy == QuantizationStrategy.GROUP.value:
                col_group = _column_groups(to_gpu(g_idx), args.group_size)
            _lib.check(
                lib.ctmi_observe_pack_quantized_gidx(
                    w.data_ptr(), _lib.dtype_code(w.dtype), rows, cols, min(blk_cols, cols), args.num_bits,
                    int(args.symmetric), _lib.ptr(col_group), packed.data_ptr(), scale.data_ptr(),
                    _lib.ptr(zero_point), _lib.stream_of(w.device),
                )
            )
        out = {"weight_shape": torch.tensor(weight.shape), "weight_packed": packed,
               "weight_scale": scale}
        if zero_point is not None:
            out["weight_zero_point"] = pack_to_int32(zero_point, args.num_bits, packed_dim=0)
        if device is not None:
            out = {k: v.to(device) for k, v in out.items()}
        return out

    def decompress_weight(
        self,
        compressed_data: Dict[str, Tensor],
        quantization_args: Optional[QuantizationArgs] = None,
    ) -> Tensor:
        args = quantization_args
        packed = to_gpu(compressed_data["weight_packed"])
        scale = to_gpu(compressed_data["weight_scale"])
        zero_point = to_gpu(compressed_data.get("weight_zero_point", None))
        g_idx = to_gpu(compressed_data.get("weight_g_idx", None))
        ws = compressed_data["weight_shape"]
        shape = torch.Size(ws.flatten().tolist() if isinstance(ws, Tensor) else [int(d) for d in ws])
        num_bits = args.num_bits
        if packed.dtype is not torch.int32:
            raise ValueError(f"Expected {torch.int32} but got {packed.dtype}, Aborting unpack.")
        if num_bits > 8:
            raise ValueError("Unpacking is only supported for less than 8 bits")

        if not args.symmetric and args.strategy in _PACKABLE:
            assert zero_point is not None, "Asymmetric quantization requires zero-point values"
            zero_point = unpack_from_int32(
                zero_point, num_bits, (shape[0], scale.shape[-1]), packed_dim=0
            )

        # dequantize(x_q, scale, zero_point, g_idx) with args=None: strategy is
        # inferred from the scale's shape, output dtype is the scale's
        carrier = _ShapeOnly(shape, torch.int8)
        dq_args = infer_dequant_args(carrier, scale)
        plan = build_qparams(carrier, scale, zero_point, dq_args, g_idx, None)
        plan.qp.qtype = _lib.QTYPE_INT
        plan.qp.num_bits = num_bits
        rows, cols = shape
        pf = 32 // num_bits
        need = math.ceil(cols / pf)
        if packed.shape[1] != need:
            packed = packed[:, :need]
        packed = packed.contiguous()
        out = torch.empty(shape, dtype=scale.dtype, device=packed.device)
        _lib.check(
            _lib.load().ctmi_pack_quantized_decompress(
                packed.data_ptr(), out.data_ptr(), _lib.dtype_code(scale.dtype), rows, cols,
                ctypes.byref(plan.qp), _lib.stream_of(packed.device),
            )
        )
        return out


class _Leftover(list):
    """(compressed entries, args) pairs the job table did not take"""
    _no_table = True


def _decompress_weights_batched(self, items) -> list:
    """PackedQuantizationCompressor.decompress_weight (pack_quantized.py:147-183) for a list
    of (compressed_data, quantization_args) pairs from one ctmi_pack_quantized_decompress_many
    call; same tensors as the per-weight calls"""
    if not items:
        return []
    if not getattr(items, "_no_table", False):
        # the common case through the job table written by columns, the rest below
        outs = _table_decompress(self, items)
        left = [k for k, out in enumerate(outs) if out is None]
        if left:
            rest = _Leftover(items[k] for k in left)
            for k, out in zip(left, _decompress_weights_batched(self, rest)):
                outs[k] = out
        return outs
    if len(items) > _CHUNK:  # the GPU starts on the first chunk while the rest is prepared
        outs = []
        for at in range(0, len(items), _CHUNK):
            outs += _decompress_weights_batched(self, _Leftover(items[at:at + _CHUNK]))
        return outs
    n = len(items)
    jobs = (_lib.WeightJob * n)()
    outs, keep, device = [], [], None
    for i, (data, args) in enumerate(items):
        packed = to_gpu(data["weight_packed"])
        scale = to_gpu(data["weight_scale"])
        zero_point = to_gpu(data.get("weight_zero_point", None))
        g_idx = to_gpu(data.get("weight_g_idx", None))
        ws = data["weight_shape"]
        shape = torch.Size(ws.flatten().tolist() if isinstance(ws, Tensor) else [int(d) for d in ws])
        if packed.dtype is not torch.int32:
            raise ValueError(f"Expected {torch.int32} but got {packed.dtype}, Aborting unpack.")
        if args.num_bits > 8:
            raise ValueError("Unpacking is only supported for less than 8 bits")
        if len(shape) != 2:
            raise ValueError(f"expected a 2-D weight, got shape {tuple(shape)}")
        if not args.symmetric and args.strategy in _PACKABLE:
            assert zero_point is not None, "Asymmetric quantization requires zero-point values"
            zero_point = unpack_from_int32(zero_point, args.num_bits, (shape[0], scale.shape[-1]),
                                           packed_dim=0)
        carrier = _ShapeOnly(shape, torch.int8)
        plan = build_qparams(carrier, scale, zero_point, infer_dequant_args(carrier, scale), g_idx, None)
        plan.qp.qtype, plan.qp.num_bits = _lib.QTYPE_INT, args.num_bits
        rows, cols = shape
        need = math.ceil(cols / (32 // args.num_bits))
        if packed.shape[1] != need:
            packed = packed[:, :need]
        packed = packed.contiguous()
        out = torch.empty(shape, dtype=scale.dtype, device=packed.device)
        j = jobs[i]
        j.src, j.dst, j.rows, j.cols = packed.data_ptr(), out.data_ptr(), rows, cols
        j.dense_dtype, j.qp = _lib.dtype_code(scale.dtype), plan.qp
        keep += [packed, plan]
        outs.append(out)
        device = device or packed.device
    _lib.check(_lib.load().ctmi_pack_quantized_decompress_many(jobs, n, _lib.stream_of(device)))
    return outs


PackedQuantizationCompressor.decompress_weights = _decompress_weights_batched


class PackedWeightBatch(LazyDenseOutputs):
    """Every weight of a state dict prepared for one-call compress / decompress.

    Holds the dense weights, their qparams, the packed outputs and the job
    tables the C ABI consumes (ctmi_pack_quantized_{compress,decompress}_many).
    Buffers are allocated once; `compress()` / `decompress()` only enqueue
    kernels, so a serving or benchmarking loop can call them repeatedly.
    """

    def __init__(self, entries, device=None, decompress_zero_points=None):
        """entries: list of dicts with keys weight, scale, quantization_args and
        optionally zero_point, g_idx (tensors on the GPU, or moved there).
        decompress_zero_points: whether decompression subtracts the zero points;
        default = only for asymmetric schemes (symmetric ones do not store any)."""
        self.n = len(entries)
        self.names = [e.get("name", str(i)) for i, e in enumerate(entries)]
        self._keep = []
        self.weights, self.packed, self.scales, self._dspecs = [], [], [], []
        self._cjobs = (_lib.WeightJob * max(self.n, 1))()
        self._djobs = (_lib.WeightJob * max(self.n, 1))()
        self.device = device
        for i, e in enumerate(entries):
            args = e["quantization_args"]
            w, scale, zp, g_idx = (to_gpu(e.get(k)) for k in ("weight", "scale", "zero_point", "g_idx"))
            if w.ndim != 2:
                raise ValueError(f"expected a 2-D weight, got shape {tuple(w.shape)}")
            if self.device is None:
                self.device = w.device
            w = w.contiguous()
            rows, cols = w.shape
            if args.num_bits > 8:
                raise ValueError("Packing is only supported for less than 8 bits")
            pf = 32 // args.num_bits
            packed = torch.empty((rows, math.ceil(cols / pf)), dtype=torch.int32, device=w.device)
            self._plan_dense((rows, cols), scale.dtype, w.device)
            cplan = build_qparams(w, scale, zp, args, g_idx, None)
            use_zp = (not args.symmetric) if decompress_zero_points is None else decompress_zero_points
            # the decompress side (its qparams, its dense output) waits for the first decompress()
            self._dspecs.append((w.shape, scale, zp if use_zp else None, g_idx, args.num_bits))
            self._keep.append(cplan)
            cj, dj = self._cjobs[i], self._djobs[i]
            cj.src, cj.dst, cj.rows, cj.cols = w.data_ptr(), packed.data_ptr(), rows, cols
            cj.dense_dtype, cj.qp = _lib.dtype_code(w.dtype), cplan.qp
            dj.src, dj.rows, dj.cols = packed.data_ptr(), rows, cols
            dj.dense_dtype = _lib.dtype_code(scale.dtype)
            self.weights.append(w)
            self.packed.append(packed)
            self.scales.append(scale)

    def _finish_decompress_job(self, i):
        shape, scale, zp, g_idx, num_bits = self._dspecs[i]
        carrier = _ShapeOnly(shape, torch.int8)
        dplan = build_qparams(carrier, scale, zp, infer_dequant_args(carrier, scale), g_idx, None)
        dplan.qp.qtype, dplan.qp.num_bits = _lib.QTYPE_INT, num_bits
        self._keep.append(dplan)
        self._djobs[i].qp = dplan.qp

    def compress(self):
        """enqueue quantize+pack of every weight; returns the packed tensors"""
        _lib.check(
            _lib.load().ctmi_pack_quantized_compress_many(self._cjobs, self.n,
                                                          _lib.stream_of(self.device))
        )
        return self.packed

    def launches(self, compress=True):
        """number of kernel launches one compress() (or decompress()) pass enqueues"""
        if not compress:
            self._ensure_dense()
        jobs = self._cjobs if compress else self._djobs
        count = _lib.load().ctmi_pack_quantized_launches(jobs, self.n, 1 if compress else 0)
        if count < 0:
            _lib.check(int(count))
        return int(count)

    def decompress(self):
        """enqueue unpack+dequantize of every packed weight; returns the dense tensors
        (allocated at the first call)"""
        dense = self._ensure_dense()
        _lib.check(
            _lib.load().ctmi_pack_quantized_decompress_many(self._djobs, self.n,
                                                            _lib.stream_of(self.device))
        )
        return dense


class ObservedWeightBatch:
    """Every weight of a model that has no scales yet, prepared for a one-call,
    one-pass compression: min-max observer, calculate_qparams, quantize and pack
    (ctmi_observe_pack_quantized_many).  Buffers are allocated once; `compress()`
    only enqueues kernels and returns, per weight, what
    PackedQuantizationCompressor.observe_and_compress_weight returns."""

    def __init__(self, entries, device=None):
        """entries: dicts with weight (2-D float tensor), quantization_args and, for
        activation ordering, g_idx.  Integer group / channel schemes of 4 or 8 bits share the
        one-pass launches; anything else (one scale per tensor, blocks, other group sizes,
        g_idx) is compressed weight by weight when compress() runs, observer first."""
        lib = _lib.load()
        self.device = device
        self.weights, self.packed, self.scales, self.zero_points, self.args = [], [], [], [], []
        self._slots = []   # per entry: ("fused", index into the job table) or ("single", entry)
        jobs = []
        for e in entries:
            args = e["quantization_args"]
            w = to_gpu(e["weight"]).contiguous()
            if w.ndim != 2:
                raise ValueError(f"expected a 2-D weight, got shape {tuple(w.shape)}")
            if self.device is None:
                self.device = w.device
            rows, cols = w.shape
            blk_cols = {QuantizationStrategy.GROUP.value: args.group_size,
                        QuantizationStrategy.CHANNEL.value: cols}.get(args.strategy, 0)
            if not (e.get("g_idx") is None and blk_cols and args.type == "int"
                    and lib.ctmi_observe_pack_quantized_supported(
                        _lib.dtype_code(w.dtype), rows, cols, blk_cols, args.num_bits)):
                self._slots.append(("single", dict(weight=w, quantization_args=args,
                                                   g_idx=e.get("g_idx"))))
                continue
            self._slots.append(("fused", len(jobs)))
            n_cells = cols // min(blk_cols, cols)
            packed = torch.empty((rows, cols * args.num_bits // 32), dtype=torch.int32, device=w.device)
            scale = torch.empty((rows, n_cells), dtype=w.dtype, device=w.device)
            zp = None if args.symmetric else torch.empty((rows, n_cells), dtype=torch.int8, device=w.device)
            jobs.append((w.data_ptr(), packed.data_ptr(), scale.data_ptr(), _lib.ptr(zp), rows, cols,
                         blk_cols, _lib.dtype_code(w.dtype), args.num_bits, int(args.symmetric)))
            self.weights.append(w)
            self.packed.append(packed)
            self.scales.append(scale)
            self.zero_points.append(zp)
            self.args.append(args)
        self.n = len(jobs)
        self._jobs = (_lib.ObservePackJob * max(self.n, 1))()
        for j, f in zip(self._jobs, jobs):
            (j.x, j.packed, j.scale, j.zero_point, j.rows, j.cols, j.blk_cols, j.x_dtype, j.num_bits,
             j.symmetric) = f

    def compress(self):
        if self.n:
            _lib.check(_lib.load().ctmi_observe_pack_quantized_many(self._jobs, self.n,
                                                                    _lib.stream_of(self.device)))
        comp = None
        out = []
        for kind, what in self._slots:
            if kind == "single":
                comp = comp or BaseCompressor.load_from_registry(CompressionFormat.pack_quantized.value)
                out.append(comp.observe_and_compress_weight(
                    what["weight"], what["quantization_args"], g_idx=what["g_idx"]))
                continue
            w, packed, scale, zp, args = (self.weights[what], self.packed[what], self.scales[what],
                                          self.zero_points[what], self.args[what])
            d = {"weight_shape": torch.tensor(w.shape), "weight_packed": packed, "weight_scale": scale}
            if zp is not None:
                d["weight_zero_point"] = pack_to_int32(zp, args.num_bits, packed_dim=0)
            out.append(d)
        return out


def _compress_state_dict_batched(self, model_state, names_to_scheme, show_progress=False,
                                 compression_device=None, precomputed=None, **kwargs):
    """BaseQuantizationCompressor.compress for pack-quantized with every weight
    handed to the C ABI in one call (same keys, dtypes and shapes as the
    per-weight loop)."""
    jobs, order = [], []

    def candidates():
        # (a generator: the first many-weight call goes out while later names are still looked at)
        for name in list(model_state.keys()):
            if not name.endswith("weight") or (precomputed is not None and name in precomputed):
                continue
            prefix = name[: -len("weight")]
            scale = model_state.get(prefix + "weight_scale", None)
            if scale is None:
                continue
            module_path = prefix[:-1] if prefix.endswith(".") else prefix
            args = names_to_scheme[module_path].weights
            weight = model_state[name]
            if model_state.get(prefix + "weight_global_scale", None) is not None:
                raise ValueError("global_scale is not supported for the PackQuantizationCompressor")
            if not can_quantize(weight, args) or weight.ndim != 2:
                continue  # handled by the per-weight path below
            job = dict(name=name, weight=weight, scale=scale,
                       zero_point=model_state.get(prefix + "weight_zero_point", None),
                       g_idx=model_state.get(prefix + "weight_g_idx", None),
                       quantization_args=args)
            jobs.append(job)
            order.append((name, prefix, args))
            yield (weight, scale, job["zero_point"], None, job["g_idx"], args)

    packed_by_name = dict(precomputed or {})  # (what the caller enqueued from the modules already)
    # the common case through the job table written by columns ...
    outs = _table_compress(self, candidates())
    left = []
    for k, out in enumerate(outs):
        if out is None:
            left.append(k)
        else:
            packed_by_name[order[k][0]] = out
    # ... the rest (asymmetric, activation-ordered, not yet on the GPU) a few launches' worth
    # of weights per call: the GPU works on one chunk while the host prepares the next
    for at in range(0, len(left), _CHUNK):
        part = left[at:at + _CHUNK]
        batch = PackedWeightBatch([jobs[k] for k in part])
        for k, packed in zip(part, batch.compress()):
            packed_by_name[order[k][0]] = packed

    def move(t):
        return t if compression_device is None else t.to(compression_device)

    out = {}
    for name in list(model_state.keys()):
        value = model_state[name]
        if name in packed_by_name:
            prefix = name[: -len("weight")]
            module_path = prefix[:-1] if prefix.endswith(".") else prefix
            args = names_to_scheme[module_path].weights
            out[prefix + "weight_shape"] = move(torch.tensor(value.shape))
            out[prefix + "weight_packed"] = move(packed_by_name[name])
            if not args.symmetric and args.strategy in _PACKABLE:
                zp = to_gpu(model_state[prefix + "weight_zero_point"])
                out[prefix + "weight_zero_point"] = move(
                    pack_to_int32(zp, args.num_bits, packed_dim=0))
        elif name.endswith("weight") and model_state.get(name[: -len("weight")] + "weight_scale") is not None:
            prefix = name[: -len("weight")]
            module_path = prefix[:-1] if prefix.endswith(".") else prefix
            single = self.compress_weight(
                weight=value, scale=model_state[prefix + "weight_scale"],
                zero_point=model_state.get(prefix + "weight_zero_point", None),
                g_idx=model_state.get(prefix + "weight_g_idx", None),
                quantization_args=names_to_scheme[module_path].weights,
                device=compression_device)
            for key, tensor in single.items():
                out[prefix + key] = move(tensor)
        elif name.endswith("zero_point") and self._skip_zp(name, names_to_scheme):
            continue
        elif name not in out:
            out[name] = move(value)
    return out


PackedQuantizationCompressor.compress = _compress_state_dict_batched


# ---------------------------------------------------------------------------------------------
# Module pathways (ModelCompressor.compress_model / decompress_model): the common case - a 2-D
# float weight on the GPU with group or channel scales, symmetric, no activation ordering - goes
# into a job table written by columns; everything else takes the state-dict path above.
_FLOAT_DTYPES = FLOAT_DTYPES
# what compression takes away from a module or writes anew (a symmetric scheme stores no zero points)
_REPLACED = ("weight", "weight_zero_point", "weight_packed", "weight_shape")
_args_key = args_key


class _CompressSpec:
    """what run_table needs for ctmi_pack_quantized_compress_many.  Records are
    (weight, scale, zero_point, global_scale, g_idx, args).  Taken: a 2-D float weight on the
    GPU, group or channel scales, symmetric, no activation ordering."""
    job_struct = _lib.WeightJob

    def __init__(self):
        self._args = {}

    def key(self, rec):
        w, scale, zp, gs, g_idx, args = rec
        k = self._args.get(id(args))
        if k is None:
            k = self._args[id(args)] = _args_key(args)
        if (gs is not None or g_idx is not None or not on_gpu(w) or w.ndim != 2 or w.numel() == 0
                or w.dtype not in _FLOAT_DTYPES or not on_gpu(scale, w.device)
                or scale.dtype not in _FLOAT_DTYPES or (zp is not None and not on_gpu(zp, w.device))
                or not k[2] or k[3] not in _PACKABLE or k[1] != "int" or not 1 <= k[0] <= 8):
            return None
        return ("c", w.shape, w.dtype, scale.shape, scale.dtype, None if zp is None else zp.dtype, k)

    def out_spec(self, rec):
        w, args = rec[0], rec[5]
        return (w.shape[0], -(-w.shape[1] // (32 // args.num_bits))), torch.int32, w.device

    def plan(self, rec):
        w, scale, zp, gs, g_idx, args = rec
        # the zero points of a symmetric scheme (all zero) take part in the arithmetic as they
        # are, as in the reference's compress_weight
        return build_qparams(w, scale, zp, args, None, None)

    def row(self, rec, out):
        w, scale, zp = rec[0], rec[1], rec[2]
        return (w.data_ptr(), out.data_ptr(), w.shape[0], w.shape[1], _lib.dtype_code(w.dtype),
                scale.data_ptr(), 0 if zp is None else zp.data_ptr(), 0, 0)


class _DecompressSpec:
    """... for ctmi_pack_quantized_decompress_many.  Records are (compressed entries of one
    weight under their local names, args).  Taken: packed words and 2-D float scales on the
    GPU, symmetric (no zero points), no activation ordering."""
    job_struct = _lib.WeightJob

    def __init__(self):
        self._shapes = {}

    def key(self, rec):
        data, args = rec
        packed, scale, ws = data.get("weight_packed"), data.get("weight_scale"), data.get("weight_shape")
        if (ws is None or not on_gpu(packed) or packed.dtype is not torch.int32 or packed.ndim != 2
                or not on_gpu(scale, packed.device) or scale.ndim != 2 or scale.dtype not in _FLOAT_DTYPES
                or not args.symmetric or args.strategy not in _PACKABLE or not 1 <= args.num_bits <= 8
                or data.get("weight_zero_point") is not None or data.get("weight_g_idx") is not None
                or (isinstance(ws, Tensor) and ws.device.type != "cpu")):
            return None
        shape = tuple(ws.flatten().tolist() if isinstance(ws, Tensor) else [int(d) for d in ws])
        if len(shape) != 2 or packed.shape != (shape[0], -(-shape[1] // (32 // args.num_bits))):
            return None
        self._shapes[id(data)] = shape
        return ("d", shape, scale.shape, scale.dtype, args.num_bits)

    def out_spec(self, rec):
        data = rec[0]
        return self._shapes[id(data)], data["weight_scale"].dtype, data["weight_packed"].device

    def plan(self, rec):
        data, args = rec
        # dequantize(x_q, scale, zero_point=None, args=None): the strategy follows from the two
        # shapes, the output dtype is the scale's (pack_quantized.py:176-181)
        scale = data["weight_scale"]
        carrier = _ShapeOnly(self._shapes[id(data)], torch.int8)
        plan = build_qparams(carrier, scale, None, infer_dequant_args(carrier, scale), None, None)
        plan.qp.qtype, plan.qp.num_bits = _lib.QTYPE_INT, args.num_bits
        return plan

    def row(self, rec, out):
        data = rec[0]
        scale = data["weight_scale"]
        shape = self._shapes[id(data)]
        return (data["weight_packed"].data_ptr(), out.data_ptr(), shape[0], shape[1],
                _lib.dtype_code(scale.dtype), scale.data_ptr(), 0, 0, 0)


def _table_compress(self, recs) -> list:
    """packed words per (weight, scale, zero_point, global_scale, g_idx, args) record from
    many-weight calls; None where the record is not one the job table takes"""
    return run_table(self, recs, _CompressSpec(), _lib.load().ctmi_pack_quantized_compress_many)


def _table_decompress(self, recs) -> list:
    """dense weights per (compressed entries, args) record; None where the table does not take it"""
    return run_table(self, recs, _DecompressSpec(), _lib.load().ctmi_pack_quantized_decompress_many)


def _compress_modules_fast(self, members, names_to_scheme) -> None:
    """PackedQuantizationCompressor.compress_modules: compress_module
    (compressors/base.py:125-151, pack_quantized.py:88-146) for every (prefix, module) pair"""
    new_param = torch.nn.Parameter
    recs = []
    for prefix, module in members:
        params = module._parameters
        recs.append((params.get("weight"), params.get("weight_scale"), params.get("weight_zero_point"),
                     params.get("weight_global_scale"), params.get("weight_g_idx"),
                     names_to_scheme[prefix].weights))
    outs = _table_compress(self, recs)
    # the kernels are enqueued: the modules get their new parameters while the GPU works
    taken = [i for i, out in enumerate(outs) if out is not None]
    if taken:
        dims = torch.tensor([tuple(recs[i][0].shape) for i in taken]).unbind(0)  # every weight_shape, one host tensor
        for i, dim in zip(taken, dims):
            params = members[i][1]._parameters
            rest = [(n, p) for n, p in params.items() if n not in _REPLACED]
            params.clear()
            params["weight_packed"] = new_param(outs[i], requires_grad=False)
            params["weight_shape"] = new_param(dim, requires_grad=False)
            params.update(rest)
    slow = [members[i] for i, out in enumerate(outs) if out is None]
    if slow:
        BaseQuantizationCompressor.compress_modules(self, slow, names_to_scheme)


def _decompress_modules_fast(self, members, names_to_scheme) -> None:
    """PackedQuantizationCompressor.decompress_modules: decompress_module
    (compressors/base.py:165-190, pack_quantized.py:147-183) for every (prefix, module) pair"""
    new_param = torch.nn.Parameter
    recs = [(module._parameters, names_to_scheme[prefix].weights) for prefix, module in members]
    outs = _table_decompress(self, recs)
    for (prefix, module), out in zip(members, outs):
        if out is not None:
            module._parameters["weight"] = new_param(out, requires_grad=False)
    slow = [members[i] for i, out in enumerate(outs) if out is None]
    if slow:
        BaseQuantizationCompressor.decompress_modules(self, slow, names_to_scheme)


PackedQuantizationCompressor.table_compress = _table_compress
PackedQuantizationCompressor.compress_modules = _compress_modules_fast
PackedQuantizationCompressor.decompress_modules = _decompress_modules_fast
