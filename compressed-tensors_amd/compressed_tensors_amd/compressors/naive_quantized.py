"""`naive-quantized` / `int-quantized` / `float-quantized`: weights stored in the
nearest torch dtype (int8 or float8_e4m3fn).

Reference: compressors/quantized_compressors/naive_quantized.py:36-154.
"""
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
    _rows_cols, _ShapeOnly, build_qparams, dequantize, infer_dequant_args, quantize,
)
from compressed_tensors_amd.quantization.helpers import can_quantize
from compressed_tensors_amd.quantization.quant_args import QuantizationArgs

__all__ = [
    "QuantizedWeightBatch",
    "observe_and_compress_weights",
    "NaiveQuantizationCompressor",
    "IntQuantizationCompressor",
    "FloatQuantizationCompressor",
]


class QuantizedWeightBatch(LazyDenseOutputs):
    """Every weight of a state dict prepared for one-call quantize / dequantize
    (ctmi_qdq_many): codes in int8 or float8_e4m3fn as the scheme says, buffers
    allocated once, `compress()` / `decompress()` only enqueue kernels."""

    _dense_field = "out"

    def __init__(self, entries, device=None):
        """entries: dicts with weight, scale, quantization_args and optionally
        zero_point, g_idx (tensors on the GPU, or moved there)"""
        self.n = len(entries)
        self.device = device
        self._keep = []
        self.weights, self.codes = [], []
        self._cjobs = (_lib.QdqJob * max(self.n, 1))()
        self._djobs = (_lib.QdqJob * max(self.n, 1))()
        for i, e in enumerate(entries):
            args = e["quantization_args"]
            w, scale, zp, g_idx = (to_gpu(e.get(k)) for k in ("weight", "scale", "zero_point", "g_idx"))
            if self.device is None:
                self.device = w.device
            w = w.contiguous()
            rows, cols = _rows_cols(w)
            codes = torch.empty(w.shape, dtype=args.pytorch_dtype(), device=w.device)
            self._plan_dense(w.shape, scale.dtype, w.device)
            cplan = build_qparams(w, scale, zp, args, g_idx, None)
            dq_args = infer_dequant_args(_ShapeOnly(w.shape, codes.dtype), scale)
            # a symmetric scheme stores no zero points: its decompression sees none
            dplan = build_qparams(_ShapeOnly(w.shape, codes.dtype), scale,
                                  None if args.symmetric else zp, dq_args, g_idx, None)
            self._keep += [cplan, dplan, scale, zp, g_idx]
            cj, dj = self._cjobs[i], self._djobs[i]
            cj.x, cj.out, cj.rows, cj.cols = w.data_ptr(), codes.data_ptr(), rows, cols
            cj.x_dtype, cj.out_dtype, cj.qp = _lib.dtype_code(w.dtype), _lib.dtype_code(codes.dtype), cplan.qp
            dj.x, dj.rows, dj.cols = codes.data_ptr(), rows, cols  # out: _ensure_dense
            dj.x_dtype, dj.out_dtype, dj.qp = _lib.dtype_code(codes.dtype), _lib.dtype_code(scale.dtype), dplan.qp
            self.weights.append(w)
            self.codes.append(codes)

    def compress(self):
        """enqueue the quantization of every weight; returns the code tensors"""
        _lib.check(_lib.load().ctmi_qdq_many(self._cjobs, self.n, 1, 0, _lib.stream_of(self.device)))
        return self.codes

    def decompress(self):
        """enqueue the dequantization of every code tensor; returns the dense tensors
        (allocated at the first call)"""
        dense = self._ensure_dense()
        _lib.check(_lib.load().ctmi_qdq_many(self._djobs, self.n, 0, 1, _lib.stream_of(self.device)))
        return dense


def observe_and_compress_weights(weights, quantization_args: QuantizationArgs):
    """observe_and_compress_weight for a list of 2-D weights that have no scales yet, from
    one call (ctmi_observe_quantize_many: rows of one length class share launches, eight
    weights at a time).  Returns one dict per weight; weights without a fused kernel take
    the single-weight path."""
    from compressed_tensors_amd.quantization.helpers import _zp_dtype
    from compressed_tensors_amd.quantization.quant_args import QuantizationStrategy

    args = quantization_args
    lib = _lib.load()
    qtype = _lib.QTYPE_INT if args.type == "int" else _lib.QTYPE_FLOAT
    results = [None] * len(weights)
    if args.strategy == QuantizationStrategy.BLOCK.value:
        return _observe_and_compress_blocks_many(weights, args, qtype)
    batch = []
    for i, weight in enumerate(weights):
        w = to_gpu(weight)
        blk_cols = 0
        if w.ndim == 2:
            if args.strategy == QuantizationStrategy.GROUP.value:
                blk_cols = args.group_size
            elif args.strategy == QuantizationStrategy.CHANNEL.value:
                blk_cols = w.shape[1]
        w = w.contiguous()
        fused = (
            blk_cols > 0 and w.numel() > 0 and can_quantize(w, args)
            and w.data_ptr() % (8 * w.element_size()) == 0
            and lib.ctmi_observe_quantize_supported(_lib.dtype_code(w.dtype), w.shape[0], w.shape[1],
                                                    blk_cols, qtype, args.num_bits)
        )
        if not fused:
            comp = BaseCompressor.load_from_registry(CompressionFormat.naive_quantized.value)
            results[i] = comp.observe_and_compress_weight(weight, args)
            continue
        rows, cols = w.shape
        n_cells = cols // min(blk_cols, cols)
        out = {"weight": torch.empty((rows, cols), dtype=args.pytorch_dtype(), device=w.device),
               "weight_scale": torch.empty((rows, n_cells), dtype=w.dtype, device=w.device)}
        if not args.symmetric:
            out["weight_zero_point"] = torch.empty((rows, n_cells), dtype=_zp_dtype(args), device=w.device)
        results[i] = out
        batch.append((w, out, blk_cols))
    if batch:
        jobs = (_lib.ObserveQuantizeJob * len(batch))()
        for job, (w, out, blk_cols) in zip(jobs, batch):
            job.x, job.codes, job.scale = w.data_ptr(), out["weight"].data_ptr(), out["weight_scale"].data_ptr()
            job.zero_point = _lib.ptr(out.get("weight_zero_point"))
            job.rows, job.cols, job.blk_cols = w.shape[0], w.shape[1], blk_cols
            job.x_dtype = _lib.dtype_code(w.dtype)
        dev = batch[0][0].device
        _lib.check(lib.ctmi_observe_quantize_many(
            jobs, len(batch), qtype, args.num_bits, int(args.symmetric), -1,
            _lib.dtype_code(_zp_dtype(args)), _lib.stream_of(dev)))
    return results


def _observe_and_compress_blocks_many(weights, args: QuantizationArgs, qtype: int):
    """the block strategy of observe_and_compress_weights: ctmi_observe_quantize_blocks_many for
    the weights whose blocks fit a workgroup's registers, the single-weight path for the rest"""
    from compressed_tensors_amd.quantization.helpers import _zp_dtype

    lib = _lib.load()
    bh, bw = args.block_structure
    results = [None] * len(weights)
    batches = {}
    for i, weight in enumerate(weights):
        w = to_gpu(weight)
        w = w.contiguous() if w.ndim == 2 else w
        if not (w.ndim == 2 and w.numel() > 0 and can_quantize(w, args)
                and w.data_ptr() % (8 * w.element_size()) == 0
                and lib.ctmi_observe_quantize_blocks_supported(
                    _lib.dtype_code(w.dtype), w.shape[0], w.shape[1], bh, bw, qtype, args.num_bits)):
            comp = BaseCompressor.load_from_registry(CompressionFormat.naive_quantized.value)
            results[i] = comp.observe_and_compress_weight(weight, args)
            continue
        rows, cols = w.shape
        out = {"weight": torch.empty((rows, cols), dtype=args.pytorch_dtype(), device=w.device),
               "weight_scale": torch.empty((rows // bh, cols // bw), dtype=w.dtype, device=w.device)}
        if not args.symmetric:
            out["weight_zero_point"] = torch.empty((rows // bh, cols // bw), dtype=_zp_dtype(args),
                                                   device=w.device)
        results[i] = out
        batches.setdefault(w.device, []).append((w, out))
    for dev, batch in batches.items():
        jobs = (_lib.ObserveQuantizeBlocksJob * len(batch))()
        for job, (w, out) in zip(jobs, batch):
            job.x, job.codes, job.scale = w.data_ptr(), out["weight"].data_ptr(), out["weight_scale"].data_ptr()
            job.zero_point = _lib.ptr(out.get("weight_zero_point"))
            job.rows, job.cols, job.blk_rows, job.blk_cols = w.shape[0], w.shape[1], bh, bw
            job.x_dtype = _lib.dtype_code(w.dtype)
        _lib.check(lib.ctmi_observe_quantize_blocks_many(
            jobs, len(batch), qtype, args.num_bits, int(args.symmetric), -1,
            _lib.dtype_code(_zp_dtype(args)), _lib.stream_of(dev)))
    return results


@BaseCompressor.register(name=CompressionFormat.naive_quantized.value)
class NaiveQuantizationCompressor(BaseQuantizationCompressor):
    @property
    def compression_param_names(self) -> Tuple[str]:
        return ("weight", "weight_scale", "weight_zero_point", "weight_g_idx")

    def compression_param_info(
        self, weight_shape: torch.Size, quantization_args: Optional[QuantizationArgs] = None
    ) -> Dict[str, Tuple[torch.Size, torch.dtype]]:
        return {"weight": (weight_shape, quantization_args.pytorch_dtype())}

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
            raise ValueError("global_scale is not supported for the NaiveQuantizationCompressor")
        weight, scale, zero_point, g_idx = (to_gpu(t) for t in (weight, scale, zero_point, g_idx))
        if can_quantize(weight, quantization_args):
            quantized = quantize(
                x=weight,
                scale=scale,
                zero_point=zero_point,
                g_idx=g_idx,
                args=quantization_args,
                dtype=quantization_args.pytorch_dtype(),
            )
        else:
            quantized = weight
        if device is not None:
            quantized = quantized.to(device)
        return {"weight": quantized}

    def observe_and_compress_weight(
        self, weight: Tensor, quantization_args: QuantizationArgs,
        device: Optional[torch.device] = None,
    ) -> Dict[str, Tensor]:
        """One-shot (round-to-nearest) compression of a weight that has no scales yet: the
        min-max observer (tests/mock_observer.py:38-113), calculate_qparams
        (quantization/utils/helpers.py:67-146) and compress_weight in one pass over the
        weight for channel and group strategies.  Returns compress_weight's dict plus
        "weight_scale" (and "weight_zero_point" for an asymmetric scheme)."""
        from compressed_tensors_amd.quantization.helpers import _zp_dtype, observe_weight_qparams
        from compressed_tensors_amd.quantization.quant_args import QuantizationStrategy

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
        qtype = _lib.QTYPE_INT if args.type == "int" else _lib.QTYPE_FLOAT
        if args.strategy == QuantizationStrategy.BLOCK.value and rows > 0 and cols > 0:
            out = self._observe_and_compress_blocks(w, args, qtype)
            if out is not None:
                return out if device is None else {k: v.to(device) for k, v in out.items()}
        fused = (
            blk_cols > 0 and can_quantize(weight, args) and rows > 0 and cols > 0
            and w.data_ptr() % (8 * w.element_size()) == 0
            and lib.ctmi_observe_quantize_supported(_lib.dtype_code(w.dtype), rows, cols, blk_cols,
                                                    qtype, args.num_bits)
        )
        if not fused:
            scale, zero_point = observe_weight_qparams(weight, args)
            out = self.compress_weight(weight, scale, args, zero_point=zero_point, device=device)
            out["weight_scale"] = scale if device is None else scale.to(device)
            if not args.symmetric:
                out["weight_zero_point"] = zero_point if device is None else zero_point.to(device)
            return out
        n_cells = cols // min(blk_cols, cols)
        codes = torch.empty((rows, cols), dtype=args.pytorch_dtype(), device=w.device)
        scale = torch.empty((rows, n_cells), dtype=w.dtype, device=w.device)
        zero_point = None
        if not args.symmetric:
            zero_point = torch.empty((rows, n_cells), dtype=_zp_dtype(args), device=w.device)
        zp_code = _lib.dtype_code(_zp_dtype(args))
        _lib.check(
            lib.ctmi_observe_quantize(
                w.data_ptr(), _lib.dtype_code(w.dtype), codes.data_ptr(), rows, cols, blk_cols, qtype,
                args.num_bits, int(args.symmetric), scale.data_ptr(), _lib.dtype_code(scale.dtype),
                _lib.ptr(zero_point), zp_code, _lib.stream_of(w.device),
            )
        )
        out = {"weight": codes, "weight_scale": scale}
        if zero_point is not None:
            out["weight_zero_point"] = zero_point
        if device is not None:
            out = {k: v.to(device) for k, v in out.items()}
        return out

    def _observe_and_compress_blocks(self, w: Tensor, args: QuantizationArgs, qtype: int):
        """block strategy: one workgroup per block, the weight read once
        (ctmi_observe_quantize_blocks); None where the layout has no such kernel"""
        from compressed_tensors_amd.quantization.helpers import _zp_dtype

        lib = _lib.load()
        rows, cols = w.shape
        bh, bw = args.block_structure
        if not (can_quantize(w, args) and w.data_ptr() % (8 * w.element_size()) == 0
                and lib.ctmi_observe_quantize_blocks_supported(
                    _lib.dtype_code(w.dtype), rows, cols, bh, bw, qtype, args.num_bits)):
            return None
        codes = torch.empty((rows, cols), dtype=args.pytorch_dtype(), device=w.device)
        scale = torch.empty((rows // bh, cols // bw), dtype=w.dtype, device=w.device)
        zero_point = None
        if not args.symmetric:
            zero_point = torch.empty((rows // bh, cols // bw), dtype=_zp_dtype(args), device=w.device)
        _lib.check(
            lib.ctmi_observe_quantize_blocks(
                w.data_ptr(), _lib.dtype_code(w.dtype), codes.data_ptr(), rows, cols, bh, bw, qtype,
                args.num_bits, int(args.symmetric), scale.data_ptr(), _lib.dtype_code(scale.dtype),
                _lib.ptr(zero_point), _lib.dtype_code(_zp_dtype(args)), _lib.stream_of(w.device),
            )
        )
        out = {"weight": codes, "weight_scale": scale}
        if zero_point is not None:
            out["weight_zero_point"] = zero_point
        return out

    def decompress_weight(
        self,
        compressed_data: Dict[str, Tensor],
        quantization_args: Optional[QuantizationArgs] = None,
    ) -> Tensor:
        return dequantize(
            x_q=to_gpu(compressed_data["weight"]),
            scale=to_gpu(compressed_data["weight_scale"]),
            zero_point=to_gpu(compressed_data.get("weight_zero_point", None)),
            g_idx=to_gpu(compressed_data.get("weight_g_idx", None)),
        )


def _compress_state_dict_batched(self, model_state, names_to_scheme, show_progress=False,
                                 compression_device=None, precomputed=None, **kwargs):
    """BaseQuantizationCompressor.compress (quantized_compressors/base.py:69-161) with
    every quantizable weight handed to the C ABI in one call: same keys, dtypes and
    values as the per-weight loop."""
    jobs, names = [], []

    def candidates():
        # (a generator: the first many-weight call goes out while later names are still looked at)
        for name in list(model_state.keys()):
            if not name.endswith("weight") or (precomputed is not None and name in precomputed):
                continue
            prefix = name[: -len("weight")]
            scale = model_state.get(prefix + "weight_scale", None)
            if scale is None:
                continue
            if model_state.get(prefix + "weight_global_scale", None) is not None:
                raise ValueError("global_scale is not supported for the NaiveQuantizationCompressor")
            module_path = prefix[:-1] if prefix.endswith(".") else prefix
            args = names_to_scheme[module_path].weights
            weight = model_state[name]
            if not can_quantize(weight, args) or weight.ndim < 1 or weight.numel() == 0:
                continue  # the per-weight path below passes it through
            job = dict(weight=weight, scale=scale, quantization_args=args,
                       zero_point=model_state.get(prefix + "weight_zero_point", None),
                       g_idx=model_state.get(prefix + "weight_g_idx", None))
            jobs.append(job)
            names.append(name)
            yield (weight, scale, job["zero_point"], None, job["g_idx"], args)

    # the common case through the job table written by columns, the rest as one batch of its own
    outs = _table_compress(self, candidates())
    codes_by_name = dict(precomputed or {})  # (what the caller enqueued from the modules already)
    codes_by_name.update((names[k], out) for k, out in enumerate(outs) if out is not None)
    left = [k for k, out in enumerate(outs) if out is None]
    if left:
        for k, codes in zip(left, QuantizedWeightBatch([jobs[k] for k in left]).compress()):
            codes_by_name[names[k]] = codes

    def move(t):
        return t if compression_device is None else t.to(compression_device)

    out = {}
    for name in list(model_state.keys()):
        value = model_state[name]
        if name in codes_by_name:
            out[name] = move(codes_by_name[name])
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
        else:
            out[name] = move(value)
    return out


NaiveQuantizationCompressor.compress = _compress_state_dict_batched


# ---------------------------------------------------------------------------------------------
# Module pathways (ModelCompressor.compress_model / decompress_model): the common case - a 2-D
# float weight on the GPU whose module holds nothing but weight, scale, zero point and bias -
# goes into a job table written by columns; everything else takes the state-dict path.
_PLAIN = ("weight", "weight_scale", "weight_zero_point", "bias")


def _plain(params) -> bool:
    """no activation ordering, no global scale, no activation qparams: nothing the table
    would have to carry besides scale and zero point"""
    for name, p in params.items():
        if p is not None and name not in _PLAIN:
            return False
    return True


class _CompressSpec:
    """what run_table needs for ctmi_qdq_many, quantizing.  Records are (weight, scale,
    zero_point, global_scale, g_idx, args).  Taken: a 2-D float weight on the GPU with float
    scales of one dimension or more, no activation ordering."""
    job_struct = _lib.QdqJob

    def __init__(self):
        self._args = {}

    def key(self, rec):
        w, scale, zp, gs, g_idx, args = rec
        k = self._args.get(id(args))
        if k is None:
            k = self._args[id(args)] = (args_key(args), args.pytorch_dtype() if args.num_bits <= 8 else None)
        if (gs is not None or g_idx is not None or not on_gpu(w) or w.ndim != 2 or w.numel() == 0
                or w.dtype not in FLOAT_DTYPES or not on_gpu(scale, w.device) or scale.ndim == 0
                or scale.dtype not in FLOAT_DTYPES or (zp is not None and not on_gpu(zp, w.device))
                or k[1] is None):
            return None
        return ("c", w.shape, w.dtype, scale.shape, scale.dtype, None if zp is None else zp.dtype, k)

    def out_spec(self, rec):
        return rec[0].shape, self._args[id(rec[5])][1], rec[0].device

    def plan(self, rec):
        w, scale, zp, gs, g_idx, args = rec
        return build_qparams(w, scale, zp, args, None, None)

    def row(self, rec, out):
        w, scale, zp = rec[0], rec[1], rec[2]
        return (w.data_ptr(), out.data_ptr(), w.shape[0], w.shape[1], _lib.dtype_code(w.dtype),
                scale.data_ptr(), 0 if zp is None else zp.data_ptr(), 0, _lib.dtype_code(out.dtype))


class _DecompressSpec:
    """... dequantizing.  Records are (compressed entries of one weight under their local
    names, args).  Taken: int8 / fp8 codes and float scales on the GPU, no activation
    ordering."""
    job_struct = _lib.QdqJob

    def key(self, rec):
        data = rec[0]
        codes, scale, zp = data.get("weight"), data.get("weight_scale"), data.get("weight_zero_point")
        if (data.get("weight_g_idx") is not None or not on_gpu(codes) or codes.ndim != 2 or codes.numel() == 0
                or codes.dtype not in (torch.int8, torch.float8_e4m3fn)
                or not on_gpu(scale, codes.device) or scale.dtype not in FLOAT_DTYPES
                or (zp is not None and not on_gpu(zp, codes.device))):
            return None
        return ("d", codes.shape, codes.dtype, scale.shape, scale.dtype, None if zp is None else zp.dtype)

    def out_spec(self, rec):
        data = rec[0]
        return data["weight"].shape, data["weight_scale"].dtype, data["weight"].device

    def plan(self, rec):
        # dequantize(x_q, scale, zero_point, g_idx=None): the strategy follows from the two
        # shapes, the output dtype is the scale's (naive_quantized.py:116-136)
        data = rec[0]
        codes, scale = data["weight"], data["weight_scale"]
        carrier = _ShapeOnly(codes.shape, codes.dtype)
        return build_qparams(carrier, scale, data.get("weight_zero_point"),
                             infer_dequant_args(carrier, scale), None, None)

    def row(self, rec, out):
        data = rec[0]
        codes, scale, zp = data["weight"], data["weight_scale"], data.get("weight_zero_point")
        return (codes.data_ptr(), out.data_ptr(), codes.shape[0], codes.shape[1], _lib.dtype_code(codes.dtype),
                scale.data_ptr(), 0 if zp is None else zp.data_ptr(), 0, _lib.dtype_code(out.dtype))


def _table_compress(self, recs) -> list:
    """codes per (weight, scale, zero_point, global_scale, g_idx, args) record from many-weight
    calls; None where the record is not one the job table takes"""
    return run_table(self, recs, _CompressSpec(), _lib.load().ctmi_qdq_many, 1, 0)


def _table_decompress(self, recs) -> list:
    """dense weights per (compressed entries, args) record; None where the table does not take it"""
    return run_table(self, recs, _DecompressSpec(), _lib.load().ctmi_qdq_many, 0, 1)


def _compress_modules_fast(self, members, names_to_scheme) -> None:
    """NaiveQuantizationCompressor.compress_modules: compress_module (compressors/base.py:125-151,
    naive_quantized.py:79-114) for every (prefix, module) pair"""
    new_param = torch.nn.Parameter
    recs, plain = [], []
    for prefix, module in members:
        params = module._parameters
        ok = _plain(params)
        plain.append(ok)
        # (a module that holds more than weight, scale, zero point and bias: the state-dict path)
        recs.append((params.get("weight") if ok else None, params.get("weight_scale"),
                     params.get("weight_zero_point"), None, None, names_to_scheme[prefix].weights))
    outs = _table_compress(self, recs)
    # the kernels are enqueued: the modules get their new parameters while the GPU works
    for (prefix, module), rec, out in zip(members, recs, outs):
        if out is not None:
            params = module._parameters
            params["weight"] = new_param(out, requires_grad=False)
            if rec[5].symmetric and rec[2] is not None:  # a symmetric scheme stores no zero points
                del params["weight_zero_point"]
    slow = [members[i] for i, out in enumerate(outs) if out is None]
    if slow:
        BaseQuantizationCompressor.compress_modules(self, slow, names_to_scheme)


def _decompress_modules_fast(self, members, names_to_scheme) -> None:
    """NaiveQuantizationCompressor.decompress_modules: decompress_module
    (compressors/base.py:165-190, naive_quantized.py:116-136) for every (prefix, module) pair"""
    new_param = torch.nn.Parameter
    recs = [(module._parameters if _plain(module._parameters) else {}, None) for _, module in members]
    outs = _table_decompress(self, recs)
    for (prefix, module), out in zip(members, outs):
        if out is not None:
            module._parameters["weight"] = new_param(out, requires_grad=False)
    slow = [members[i] for i, out in enumerate(outs) if out is None]
    if slow:
        BaseQuantizationCompressor.decompress_modules(self, slow, names_to_scheme)


def _decompress_weights_batched(self, items) -> list:
    """NaiveQuantizationCompressor.decompress_weight for a list of (compressed_data,
    quantization_args) pairs: many-weight calls where the job table takes them"""
    outs = _table_decompress(self, items)
    for k, out in enumerate(outs):
        if out is None:
            outs[k] = self.decompress_weight(compressed_data=items[k][0], quantization_args=items[k][1])
    return outs


NaiveQuantizationCompressor.decompress_weights = _decompress_weights_batched
NaiveQuantizationCompressor.table_compress = _table_compress
NaiveQuantizationCompressor.compress_modules = _compress_modules_fast
NaiveQuantizationCompressor.decompress_modules = _decompress_modules_fast


@BaseCompressor.register(name=CompressionFormat.int_quantized.value)
class IntQuantizationCompressor(NaiveQuantizationCompressor):
    pass


@BaseCompressor.register(name=CompressionFormat.float_quantized.value)
class FloatQuantizationCompressor(NaiveQuantizationCompressor):
    pass
