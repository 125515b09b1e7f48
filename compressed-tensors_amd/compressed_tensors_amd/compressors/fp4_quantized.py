"""`nvfp4-pack-quantized`: e2m1 codes, two per byte.

Reference: compressors/quantized_compressors/fp4_quantized.py
(NVFP4PackedCompressor :44-123, pack_fp4_to_uint8 :135-178,
unpack_fp4_from_uint8 :187-221).
"""
import ctypes
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
    build_qparams,
    infer_dequant_args,
)
from compressed_tensors_amd.quantization.quant_args import QuantizationArgs

__all__ = [
    "nvfp4_observe_and_compress_weights",
    "Fp4WeightBatch",
    "NVFP4PackedCompressor",
    "MXFP4PackedCompressor",
    "pack_fp4_to_uint8",
    "unpack_fp4_from_uint8",
    "FLOAT_TO_E2M1",
]

FLOAT_TO_E2M1 = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
_FLOATS = (torch.float32, torch.float16, torch.bfloat16)


def pack_fp4_to_uint8(x: Tensor) -> Tensor:
    """[m, n] e2m1-valued tensor -> uint8 [m, n/2]; low nibble first, sign in bit 3."""
    m, n = x.shape
    if n % 2 != 0:
        raise ValueError("tensor must have an even number of columns for nvfp4 compression")
    x = to_gpu(x).contiguous()
    if x.dtype not in _FLOATS:
        raise NotImplementedError(f"fp4 packing of dtype {x.dtype} is not supported")
    out = torch.empty((m, n // 2), dtype=torch.uint8, device=x.device)
    _lib.check(
        _lib.load().ctmi_pack_fp4_to_uint8(
            x.data_ptr(), _lib.dtype_code(x.dtype), out.data_ptr(), m, n,
            _lib.stream_of(x.device),
        )
    )
    return out


def unpack_fp4_from_uint8(
    a: Tensor, m: int, n: int, dtype: Optional[torch.dtype] = torch.bfloat16
) -> Tensor:
    """uint8 [m, n/2] -> [m, n] of `dtype`"""
    assert a.dtype == torch.uint8
    a = to_gpu(a).contiguous()
    if a.numel() * 2 != m * n:
        raise RuntimeError(f"cannot unpack {a.numel()} bytes into [{m}, {n}]")
    out = torch.empty((m, n), dtype=dtype, device=a.device)
    _lib.check(
        _lib.load().ctmi_unpack_fp4_from_uint8(
            a.data_ptr(), out.data_ptr(), _lib.dtype_code(dtype), m, n, _lib.stream_of(a.device)
        )
    )
    return out


@BaseCompressor.register(name=CompressionFormat.nvfp4_pack_quantized.value)
class NVFP4PackedCompressor(BaseQuantizationCompressor):
    @property
    def compression_param_names(self) -> Tuple[str]:
        return ("weight_packed", "weight_scale", "weight_zero_point", "weight_global_scale")

    def compression_param_info(
        self, weight_shape: torch.Size, quantization_args: Optional[QuantizationArgs] = None
    ) -> Dict[str, Tuple[torch.Size, torch.dtype]]:
        return {
            "weight_packed": (torch.Size((weight_shape[0], weight_shape[1] // 2)), torch.uint8)
        }

    def compress_weight(
        self,
        weight: Tensor,
        scale: Tensor,
        global_scale: Tensor,
        quantization_args: QuantizationArgs,
        device: Optional[torch.device] = None,
        zero_point: Optional[Tensor] = None,
        g_idx: Optional[Tensor] = None,
    ) -> Dict[str, Tensor]:
        weight, scale, global_scale, zero_point = (
            to_gpu(t) for t in (weight, scale, global_scale, zero_point)
        )
        if weight.ndim != 2:
            raise ValueError(f"expected a 2-D weight, got shape {tuple(weight.shape)}")
        # the reference does not forward g_idx to quantize()
        plan = build_qparams(weight, scale, zero_point, quantization_args, None, global_scale)
        w = weight.contiguous()
        rows, cols = w.shape
        if cols % 2 != 0:
            raise ValueError("tensor must have an even number of columns for nvfp4 compression")
        packed = torch.empty((rows, cols // 2), dtype=torch.uint8, device=w.device)
        _lib.check(
            _lib.load().ctmi_nvfp4_compress(
                w.data_ptr(), _lib.dtype_code(w.dtype), packed.data_ptr(), rows, cols,
                ctypes.byref(plan.qp), _lib.stream_of(w.device),
            )
        )
        if device is not None:
            packed = packed.to(device)
        return {"weight_packed": packed}

    def observe_and_compress_weight(
        self, weight: Tensor, quantization_args: QuantizationArgs,
        global_scale: Optional[Tensor] = None, device: Optional[torch.device] = None,
    ) -> Dict[str, Tensor]:
        """One-shot compression of a weight that has no scales yet: the global scale
        (generate_gparam of the tensor's min / max, helpers.py:414-434, unless given),
        then the group scales of the min-max observer and compress_weight in one pass
        over the weight.  Returns weight_packed, weight_scale and weight_global_scale."""
        from compressed_tensors_amd.quantization.helpers import generate_gparam, minmax

        args = quantization_args
        weight = to_gpu(weight)
        if weight.ndim != 2:
            raise ValueError(f"expected a 2-D weight, got shape {tuple(weight.shape)}")
        w = weight.contiguous()
        rows, cols = w.shape
        if args.group_size != 16 or cols % 16 or w.data_ptr() % (8 * w.element_size()):
            raise NotImplementedError("one-pass nvfp4 compression needs groups of 16 columns")
        if global_scale is None:
            mn, mx = minmax(w, rows, cols)
            global_scale = generate_gparam(mn.reshape(1), mx.reshape(1))
        gs = to_gpu(global_scale).to(torch.float32).reshape(-1).contiguous()
        packed = torch.empty((rows, cols // 2), dtype=torch.uint8, device=w.device)
        scale = torch.empty((rows, cols // 16), dtype=torch.float8_e4m3fn, device=w.device)
        _lib.check(
            _lib.load().ctmi_observe_nvfp4_compress(
                w.data_ptr(), _lib.dtype_code(w.dtype), rows, cols, gs.data_ptr(),
                packed.data_ptr(), scale.data_ptr(), _lib.stream_of(w.device),
            )
        )
        out = {"weight_packed": packed, "weight_scale": scale, "weight_global_scale": gs}
        if device is not None:
            out = {k: v.to(device) for k, v in out.items()}
        return out

    def decompress_weight(
        self,
        compressed_data: Dict[str, Tensor],
        quantization_args: Optional[QuantizationArgs] = None,
    ) -> Tensor:
        packed = to_gpu(compressed_data["weight_packed"]).contiguous()
        scale = to_gpu(compressed_data["weight_scale"])
        global_scale = to_gpu(compressed_data["weight_global_scale"])
        assert packed.dtype == torch.uint8
        m, half = packed.shape
        shape = torch.Size((m, half * 2))
        # unpack to bf16, then dequantize(x_q, scale, global_scale, dtype=bf16) with
        # the strategy inferred from the scale's shape
        carrier = _ShapeOnly(shape, torch.bfloat16)
        dq_args = infer_dequant_args(carrier, scale)
        plan = build_qparams(carrier, scale, None, dq_args, None, global_scale)
        plan.qp.qtype = _lib.QTYPE_FLOAT
        plan.qp.num_bits = 4
        # only the group path of the reference honours the requested bf16 output
        out_dtype = torch.bfloat16 if plan.grouped else plan.dequant_dtype
        out = torch.empty(shape, dtype=out_dtype, device=packed.device)
        _lib.check(
            _lib.load().ctmi_nvfp4_decompress(
                packed.data_ptr(), out.data_ptr(), _lib.dtype_code(out_dtype), shape[0], shape[1],
                ctypes.byref(plan.qp), _lib.stream_of(packed.device),
            )
        )
        return out


def nvfp4_observe_and_compress_weights(weights, quantization_args: QuantizationArgs,
                                       global_scales=None):
    """NVFP4PackedCompressor.observe_and_compress_weight for a list of 2-D weights from one
    call (ctmi_observe_nvfp4_compress_many: weights of one dtype share launches, eight at a
    time).  global_scales: one per weight, or None (then each is generate_gparam of its
    weight's min / max).  Returns one dict per weight."""
    from compressed_tensors_amd.quantization.helpers import generate_gparam, minmax

    args = quantization_args
    if args.group_size != 16:
        raise NotImplementedError("one-pass nvfp4 compression needs groups of 16 columns")
    ws = [to_gpu(w).contiguous() for w in weights]
    jobs = (_lib.ObserveNvfp4Job * max(len(ws), 1))()
    results = []
    for i, (job, w) in enumerate(zip(jobs, ws)):
        if w.ndim != 2:
            raise ValueError(f"expected a 2-D weight, got shape {tuple(w.shape)}")
        rows, cols = w.shape
        if cols % 16 or w.data_ptr() % (8 * w.element_size()):
            raise NotImplementedError("one-pass nvfp4 compression needs groups of 16 columns")
        gs = None if global_scales is None else global_scales[i]
        if gs is None:
            mn, mx = minmax(w, rows, cols)
            gs = generate_gparam(mn.reshape(1), mx.reshape(1))
        gs = to_gpu(gs).to(torch.float32).reshape(-1).contiguous()
        packed = torch.empty((rows, cols // 2), dtype=torch.uint8, device=w.device)
        scale = torch.empty((rows, cols // 16), dtype=torch.float8_e4m3fn, device=w.device)
        job.x, job.global_scale, job.packed, job.scale = (
            w.data_ptr(), gs.data_ptr(), packed.data_ptr(), scale.data_ptr())
        job.rows, job.cols, job.x_dtype = rows, cols, _lib.dtype_code(w.dtype)
        results.append({"weight_packed": packed, "weight_scale": scale, "weight_global_scale": gs})
    if ws:
        _lib.check(_lib.load().ctmi_observe_nvfp4_compress_many(jobs, len(ws), _lib.stream_of(ws[0].device)))
    return results


class Fp4WeightBatch(LazyDenseOutputs):
    """Every nvfp4 weight of a state dict prepared for one-call compress / decompress
    (ctmi_nvfp4_{compress,decompress}_many).  Buffers are allocated once; `compress()`
    and `decompress()` only enqueue kernels."""

    def __init__(self, entries):
        """entries: dicts with keys weight, scale (fp8 group scales), global_scale,
        quantization_args, optionally zero_point"""
        self.n = len(entries)
        self._keep = []
        self.weights, self.packed = [], []
        self._cjobs = (_lib.WeightJob * max(self.n, 1))()
        self._djobs = (_lib.WeightJob * max(self.n, 1))()
        self.device = None
        for i, e in enumerate(entries):
            args = e["quantization_args"]
            w, scale, gs, zp = (to_gpu(e.get(k)) for k in ("weight", "scale", "global_scale", "zero_point"))
            if w.ndim != 2:
                raise ValueError(f"expected a 2-D weight, got shape {tuple(w.shape)}")
            if self.device is None:
                self.device = w.device
            w = w.contiguous()
            rows, cols = w.shape
            if cols % 2 != 0:
                raise ValueError("tensor must have an even number of columns for nvfp4 compression")
            packed = torch.empty((rows, cols // 2), dtype=torch.uint8, device=w.device)
            cplan = build_qparams(w, scale, zp, args, None, gs)
            carrier = _ShapeOnly(w.shape, torch.bfloat16)
            dq_args = infer_dequant_args(carrier, scale)
            dplan = build_qparams(carrier, scale, None, dq_args, None, gs)
            dplan.qp.qtype, dplan.qp.num_bits = _lib.QTYPE_FLOAT, 4
            out_dtype = torch.bfloat16 if dplan.grouped else dplan.dequant_dtype
            self._plan_dense((rows, cols), out_dtype, w.device)
            self._keep += [cplan, dplan]
            cj, dj = self._cjobs[i], self._djobs[i]
            cj.src, cj.dst, cj.rows, cj.cols = w.data_ptr(), packed.data_ptr(), rows, cols
            cj.dense_dtype, cj.qp = _lib.dtype_code(w.dtype), cplan.qp
            dj.src, dj.rows, dj.cols = packed.data_ptr(), rows, cols  # dst: _ensure_dense
            dj.dense_dtype, dj.qp = _lib.dtype_code(out_dtype), dplan.qp
            self.weights.append(w)
            self.packed.append(packed)

    def compress(self):
        """enqueue quantize + pack of every weight; returns the packed tensors"""
        if self.n:
            _lib.check(_lib.load().ctmi_nvfp4_compress_many(self._cjobs, self.n, _lib.stream_of(self.device)))
        return self.packed

    def decompress(self):
        """enqueue unpack + dequantize of every packed weight; returns the dense tensors
        (allocated at the first call)"""
        dense = self._ensure_dense()
        if self.n:
            _lib.check(_lib.load().ctmi_nvfp4_decompress_many(self._djobs, self.n, _lib.stream_of(self.device)))
        return dense


def _compress_state_dict_batched(self, model_state, names_to_scheme, show_progress=False,
                                 compression_device=None, precomputed=None, **kwargs):
    """BaseQuantizationCompressor.compress (quantized_compressors/base.py:69-161) with
    every nvfp4 weight handed to the C ABI in one call: same keys, dtypes and values as
    the per-weight loop."""
    jobs, names = [], []

    def candidates():
        # (a generator: the first many-weight call goes out while later names are still looked at)
        for name in list(model_state.keys()):
            if not name.endswith("weight") or (precomputed is not None and name in precomputed):
                continue
            prefix = name[: -len("weight")]
            scale = model_state.get(prefix + "weight_scale", None)
            gs = model_state.get(prefix + "weight_global_scale", None)
            weight = model_state[name]
            if scale is None or gs is None or weight.ndim != 2 or weight.numel() == 0:
                continue  # the per-weight path below deals with it (or raises as the reference does)
            module_path = prefix[:-1] if prefix.endswith(".") else prefix
            job = dict(weight=weight, scale=scale, global_scale=gs,
                       zero_point=model_state.get(prefix + "weight_zero_point", None),
                       quantization_args=names_to_scheme[module_path].weights)
            jobs.append(job)
            names.append(name)
            yield (weight, scale, job["zero_point"], gs, None, job["quantization_args"])

    # the common case through the job table written by columns, the rest as one batch of its own
    outs = _table_compress(self, candidates())
    packed_by_name = dict(precomputed or {})  # (what the caller enqueued from the modules already)
    packed_by_name.update((names[k], out) for k, out in enumerate(outs) if out is not None)
    left = [k for k, out in enumerate(outs) if out is None]
    if left:
        for k, packed in zip(left, Fp4WeightBatch([jobs[k] for k in left]).compress()):
            packed_by_name[names[k]] = packed

    def move(t):
        return t if compression_device is None else t.to(compression_device)

    out = {}
    for name in list(model_state.keys()):
        value = model_state[name]
        prefix = name[: -len("weight")] if name.endswith("weight") else None
        if name in packed_by_name:
            out[prefix + "weight_packed"] = move(packed_by_name[name])
        elif prefix is not None and model_state.get(prefix + "weight_scale") is not None:
            module_path = prefix[:-1] if prefix.endswith(".") else prefix
            single = self.compress_weight(
                weight=value, scale=model_state[prefix + "weight_scale"],
                global_scale=model_state.get(prefix + "weight_global_scale", None),
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


NVFP4PackedCompressor.compress = _compress_state_dict_batched


# ---------------------------------------------------------------------------------------------
# Module pathways (ModelCompressor.compress_model / decompress_model): a 2-D float weight on the
# GPU with fp8 group scales and an fp32 global scale goes into a job table written by columns;
# everything else takes the state-dict path.
_OWN = ("weight", "weight_packed", "weight_scale", "weight_zero_point", "weight_global_scale", "bias")
_SCALE_DTYPES = FLOAT_DTYPES + (torch.float8_e4m3fn,)


def _own_only(params) -> bool:
    for name, p in params.items():
        if p is not None and name not in _OWN:
            return False
    return True


class _CompressSpec:
    """what run_table needs for ctmi_nvfp4_compress_many.  Records are (weight, scale,
    zero_point, global_scale, g_idx, args); the reference does not forward g_idx to quantize().
    Taken: a 2-D float weight on the GPU with 2-D scales and an fp32 global scale of one value."""
    job_struct = _lib.WeightJob

    def __init__(self):
        self._args = {}

    def key(self, rec):
        w, scale, zp, gs, g_idx, args = rec
        if (not on_gpu(w) or w.ndim != 2 or w.numel() == 0 or w.shape[1] % 2 or w.dtype not in FLOAT_DTYPES
                or not on_gpu(scale, w.device) or scale.dtype not in _SCALE_DTYPES or scale.ndim != 2
                or not on_gpu(gs, w.device) or gs.dtype is not torch.float32 or gs.numel() != 1
                or (zp is not None and not on_gpu(zp, w.device))):
            return None
        k = self._args.get(id(args))
        if k is None:
            k = self._args[id(args)] = args_key(args)
        return ("c", w.shape, w.dtype, scale.shape, scale.dtype, None if zp is None else zp.dtype, k)

    def out_spec(self, rec):
        w = rec[0]
        return (w.shape[0], w.shape[1] // 2), torch.uint8, w.device

    def plan(self, rec):
        w, scale, zp, gs, g_idx, args = rec
        return build_qparams(w, scale, zp, args, None, gs)

    def row(self, rec, out):
        w, scale, zp, gs = rec[0], rec[1], rec[2], rec[3]
        return (w.data_ptr(), out.data_ptr(), w.shape[0], w.shape[1], _lib.dtype_code(w.dtype),
                scale.data_ptr(), 0 if zp is None else zp.data_ptr(), gs.data_ptr(), 0)


class _DecompressSpec:
    """... for ctmi_nvfp4_decompress_many.  Records are (compressed entries of one weight under
    their local names, args).  Taken: packed bytes, several group scales per row and an fp32
    global scale on the GPU (the reference's group path, which honours the bf16 it asks for)."""
    job_struct = _lib.WeightJob

    def key(self, rec):
        data = rec[0]
        packed, scale, gs = data.get("weight_packed"), data.get("weight_scale"), data.get("weight_global_scale")
        if (not on_gpu(packed) or packed.dtype is not torch.uint8 or packed.ndim != 2 or packed.numel() == 0
                or not on_gpu(scale, packed.device) or scale.dtype not in _SCALE_DTYPES
                or scale.ndim != 2 or scale.shape[0] != packed.shape[0] or scale.shape[1] <= 1
                or (2 * packed.shape[1]) % scale.shape[1]
                or not on_gpu(gs, packed.device) or gs.dtype is not torch.float32 or gs.numel() != 1):
            return None
        return ("d", packed.shape, scale.shape, scale.dtype)

    def out_spec(self, rec):
        packed = rec[0]["weight_packed"]
        return (packed.shape[0], 2 * packed.shape[1]), torch.bfloat16, packed.device

    def plan(self, rec):
        data = rec[0]
        packed, scale = data["weight_packed"], data["weight_scale"]
        carrier = _ShapeOnly(torch.Size((packed.shape[0], 2 * packed.shape[1])), torch.bfloat16)
        plan = build_qparams(carrier, scale, None, infer_dequant_args(carrier, scale), None,
                             data["weight_global_scale"])
        if not plan.grouped:
            raise RuntimeError(f"group scales expected, got shape {tuple(scale.shape)}")
        plan.qp.qtype, plan.qp.num_bits = _lib.QTYPE_FLOAT, 4
        return plan

    def row(self, rec, out):
        data = rec[0]
        packed = data["weight_packed"]
        return (packed.data_ptr(), out.data_ptr(), packed.shape[0], 2 * packed.shape[1],
                _lib.dtype_code(torch.bfloat16), data["weight_scale"].data_ptr(), 0,
                data["weight_global_scale"].data_ptr(), 0)


def _table_compress(self, recs) -> list:
    """packed bytes per (weight, scale, zero_point, global_scale, g_idx, args) record from
    many-weight calls; None where the record is not one the job table takes"""
    return run_table(self, recs, _CompressSpec(), _lib.load().ctmi_nvfp4_compress_many)


def _table_decompress(self, recs) -> list:
    """dense weights per (compressed entries, args) record; None where the table does not take it"""
    return run_table(self, recs, _DecompressSpec(), _lib.load().ctmi_nvfp4_decompress_many)


def _compress_modules_fast(self, members, names_to_scheme) -> None:
    """NVFP4PackedCompressor.compress_modules: compress_module (compressors/base.py:125-151,
    fp4_quantized.py:84-106) for every (prefix, module) pair"""
    new_param = torch.nn.Parameter
    recs = []
    for prefix, module in members:
        params = module._parameters
        ok = _own_only(params)
        recs.append((params.get("weight") if ok else None, params.get("weight_scale"),
                     params.get("weight_zero_point"), params.get("weight_global_scale"), None,
                     names_to_scheme[prefix].weights))
    outs = _table_compress(self, recs)
    # the kernels are enqueued: the modules get their new parameters while the GPU works
    for (prefix, module), rec, out in zip(members, recs, outs):
        if out is not None:
            params = module._parameters
            symmetric = rec[5].symmetric
            rest = [(n, p) for n, p in params.items()
                    if n not in ("weight", "weight_packed") and not (n == "weight_zero_point" and symmetric)]
            params.clear()
            params["weight_packed"] = new_param(out, requires_grad=False)
            params.update(rest)
    slow = [members[i] for i, out in enumerate(outs) if out is None]
    if slow:
        BaseQuantizationCompressor.compress_modules(self, slow, names_to_scheme)


def _decompress_modules_fast(self, members, names_to_scheme) -> None:
    """NVFP4PackedCompressor.decompress_modules: decompress_module (compressors/base.py:165-190,
    fp4_quantized.py:108-123) for every (prefix, module) pair"""
    new_param = torch.nn.Parameter
    recs = []
    for _, module in members:
        params = module._parameters
        ok = _own_only(params) and params.get("weight_zero_point") is None
        recs.append((params if ok else {}, None))
    outs = _table_decompress(self, recs)
    for (prefix, module), out in zip(members, outs):
        if out is not None:
            module._parameters["weight"] = new_param(out, requires_grad=False)
    slow = [members[i] for i, out in enumerate(outs) if out is None]
    if slow:
        BaseQuantizationCompressor.decompress_modules(self, slow, names_to_scheme)


def _decompress_weights_batched(self, items) -> list:
    """NVFP4PackedCompressor.decompress_weight for a list of (compressed_data,
    quantization_args) pairs: many-weight calls where the job table takes them"""
    outs = _table_decompress(self, items)
    for k, out in enumerate(outs):
        if out is None:
            outs[k] = self.decompress_weight(compressed_data=items[k][0], quantization_args=items[k][1])
    return outs


NVFP4PackedCompressor.decompress_weights = _decompress_weights_batched
NVFP4PackedCompressor.table_compress = _table_compress
NVFP4PackedCompressor.compress_modules = _compress_modules_fast
NVFP4PackedCompressor.decompress_modules = _decompress_modules_fast


@BaseCompressor.register(name=CompressionFormat.mxfp4_pack_quantized.value)
class MXFP4PackedCompressor(NVFP4PackedCompressor):
    pass
