"""Quantization parameter helpers on the GPU.

Signatures follow the reference's quantization/utils/helpers.py:
calculate_qparams :67-146, compute_dynamic_scales_and_zp :149-205,
calculate_range :208-234, can_quantize :373-390, generate_gparam :414-434,
strategy_cdiv :437-457.  Reductions and the qparam arithmetic run in HIP
kernels (csrc/observer.hip); shapes and dtypes of the results match the
reference's.
"""
import logging
import math
from typing import Optional, Tuple

import torch

from compressed_tensors_amd import _lib
from compressed_tensors_amd.quantization.quant_args import (
    FP4_E2M1_DATA,
    FP8_DTYPE,
    FP8_E4M3_DATA,
    QuantizationArgs,
    QuantizationStrategy,
    QuantizationType,
)

__all__ = [
    "is_fp4",
    "calculate_range",
    "calculate_qparams",
    "compute_dynamic_scales_and_zp",
    "dynamic_fake_quantize",
    "generate_gparam",
    "observe_weight_qparams",
    "observe_weights_qparams",
    "minmax",
    "can_quantize",
    "get_torch_bit_depth",
    "strategy_cdiv",
    "KV_CACHE_TARGETS",
    "is_kv_cache_quant_scheme",
]

_LOGGER = logging.getLogger(__name__)
_FLOATS = (torch.float32, torch.float16, torch.bfloat16)

KV_CACHE_TARGETS = ["re:.*self_attn$"]


def is_kv_cache_quant_scheme(scheme) -> bool:
    """does a scheme name the attention modules whose keys and values go into the cache
    (helpers.py:394-411)"""
    return any(target in KV_CACHE_TARGETS for target in scheme.targets)


def is_fp4(quantization_args: QuantizationArgs) -> bool:
    return quantization_args.num_bits == 4 and quantization_args.type == QuantizationType.FLOAT.value


def calculate_range(quantization_args: QuantizationArgs, device) -> Tuple[torch.Tensor, torch.Tensor]:
    """(q_min, q_max) as 0-d fp32 tensors on `device`."""
    if quantization_args.type == QuantizationType.INT.value:
        bit_range = 2**quantization_args.num_bits
        q_max, q_min = bit_range / 2 - 1, -bit_range / 2
    elif quantization_args.type == QuantizationType.FLOAT.value:
        if quantization_args.num_bits == 8:
            q_max, q_min = FP8_E4M3_DATA.max, FP8_E4M3_DATA.min
        elif quantization_args.num_bits == 4:
            q_max, q_min = FP4_E2M1_DATA.max, FP4_E2M1_DATA.min
        else:
            raise NotImplementedError("Range calculation only supported for 4 and 8 bits")
    else:
        raise ValueError(f"Invalid quantization type {quantization_args.type}")
    return torch.tensor(q_min, device=device), torch.tensor(q_max, device=device)


def _qtype(args: QuantizationArgs) -> int:
    return _lib.QTYPE_INT if args.type == QuantizationType.INT.value else _lib.QTYPE_FLOAT


def _zp_dtype(args: QuantizationArgs) -> torch.dtype:
    return FP8_DTYPE if is_fp4(args) else args.pytorch_dtype()


def _scale_dtype(args: QuantizationArgs, mm_dtype: torch.dtype, has_global: bool) -> torch.dtype:
    if is_fp4(args) and args.symmetric and has_global:
        return FP8_DTYPE
    return mm_dtype


def _gscale_ptr(global_scale: Optional[torch.Tensor], keep: list) -> Optional[int]:
    if global_scale is None:
        return None
    gs = global_scale.to(torch.float32).reshape(-1).contiguous()
    if gs.numel() != 1:
        raise NotImplementedError("global_scale must hold a single value")
    keep.append(gs)
    return gs.data_ptr()


def calculate_qparams(
    min_vals: torch.Tensor,
    max_vals: torch.Tensor,
    quantization_args: QuantizationArgs,
    global_scale: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Scales and zero points from per-slice minima / maxima (helpers.py:67-146)."""
    args = quantization_args
    _lib.require_gpu(min_vals, max_vals, global_scale)
    if min_vals.dtype not in _FLOATS:
        raise NotImplementedError(f"min/max of dtype {min_vals.dtype} are not supported")
    if not args.symmetric and is_fp4(args):
        raise NotImplementedError("Asymmetric Quantization is not supported for FP4")
    mn = min_vals.contiguous()
    mx = max_vals.to(min_vals.dtype).contiguous()
    keep = []
    gs_ptr = _gscale_ptr(global_scale if is_fp4(args) and args.symmetric else None, keep)
    scale_dtype = _scale_dtype(args, mn.dtype, gs_ptr is not None)
    zp_dtype = _zp_dtype(args)
    scales = torch.empty(mn.shape, dtype=scale_dtype, device=mn.device)
    zps = torch.empty(mn.shape, dtype=zp_dtype, device=mn.device)
    _lib.check(
        _lib.load().ctmi_calculate_qparams(
            mn.data_ptr(), mx.data_ptr(), _lib.dtype_code(mn.dtype), int(mn.ndim == 0),
            mn.numel(), _qtype(args), args.num_bits, int(args.symmetric), gs_ptr,
            scales.data_ptr(), _lib.dtype_code(scale_dtype), zps.data_ptr(),
            _lib.dtype_code(zp_dtype), _lib.stream_of(mn.device),
        )
    )
    if scales.ndim == 0:
        scales, zps = scales.reshape(1), zps.reshape(1)
    return scales, zps


def minmax(
    value: torch.Tensor, blk_rows: int, blk_cols: int
) -> Tuple[torch.Tensor, torch.Tensor]:
    """amin / amax over [blk_rows x blk_cols] cells of `value` viewed as
    [rows, last_dim]; returns two [ceil(rows/blk_rows), ceil(cols/blk_cols)] tensors."""
    _lib.require_gpu(value)
    v = value.contiguous()
    cols = v.shape[-1]
    rows = v.numel() // cols
    lib = _lib.load()
    out_shape = (math.ceil(rows / blk_rows), math.ceil(cols / blk_cols))
    mn = torch.empty(out_shape, dtype=v.dtype, device=v.device)
    mx = torch.empty(out_shape, dtype=v.dtype, device=v.device)
    code = _lib.dtype_code(v.dtype)
    tmp_bytes = lib.ctmi_minmax_tmp_bytes(rows, cols, blk_rows, blk_cols, code)
    tmp = torch.empty(max(tmp_bytes, 1), dtype=torch.uint8, device=v.device)
    _lib.check(
        lib.ctmi_minmax(v.data_ptr(), code, rows, cols, blk_rows, blk_cols, mn.data_ptr(),
                        mx.data_ptr(), tmp.data_ptr(), _lib.stream_of(v.device))
    )
    return mn, mx


def _observe_rows(
    value: torch.Tensor,
    blk_cols: int,
    args: QuantizationArgs,
    global_scale: Optional[torch.Tensor],
    out_shape,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """fused min/max + calculate_qparams for cells that are one row tall"""
    v = value.contiguous()
    cols = v.shape[-1]
    rows = v.numel() // cols
    keep = []
    gs_ptr = _gscale_ptr(global_scale if is_fp4(args) and args.symmetric else None, keep)
    scale_dtype = _scale_dtype(args, v.dtype, gs_ptr is not None)
    zp_dtype = _zp_dtype(args)
    scales = torch.empty(out_shape, dtype=scale_dtype, device=v.device)
    zps = torch.empty(out_shape, dtype=zp_dtype, device=v.device)
    _lib.check(
        _lib.load().ctmi_observe_qparams(
            v.data_ptr(), _lib.dtype_code(v.dtype), rows, cols, blk_cols, _qtype(args),
            args.num_bits, int(args.symmetric), gs_ptr, scales.data_ptr(),
            _lib.dtype_code(scale_dtype), zps.data_ptr(), _lib.dtype_code(zp_dtype), None, None,
            _lib.stream_of(v.device),
        )
    )
    return scales, zps


def dynamic_fake_quantize(
    value: torch.Tensor,
    args: QuantizationArgs,
    global_scale: Optional[torch.Tensor] = None,
    return_qparams: bool = False,
):
    """compute_dynamic_scales_and_zp (helpers.py:149-205) followed by fake_quantize
    (forward.py:150-189) in one pass over `value` (ctmi_dynamic_qdq).  Returns None
    when the layout has no fused kernel; the caller then makes the two calls."""
    _lib.require_gpu(value)
    if value.dtype not in _FLOATS or value.numel() == 0:
        return None
    strategy = args.strategy
    if strategy == QuantizationStrategy.TOKEN.value:
        if value.ndim <= 2:
            return None  # one scale for the whole tensor: two passes by nature
        rows = value.shape[0] * value.shape[1]
        cols = value.numel() // rows
        blk_cols = cols
        out_shape = (value.shape[0], value.shape[1]) + (1,) * (value.ndim - 2)
    elif strategy in (QuantizationStrategy.TENSOR_GROUP.value, QuantizationStrategy.GROUP.value):
        cols = value.shape[-1]
        blk_cols = args.group_size
        if value.ndim < 1 or cols % blk_cols:
            return None
        rows = value.numel() // cols
        out_shape = tuple(value.shape[:-1]) + (cols // blk_cols,)
    else:
        return None
    fp4 = is_fp4(args)
    if fp4 and not args.symmetric:
        return None
    if (global_scale is not None) != fp4:
        return None  # a global scale that calculate_qparams ignores, or fp4 without one
    lib = _lib.load()
    if not lib.ctmi_dynamic_qdq_supported(_lib.dtype_code(value.dtype), rows, cols, blk_cols,
                                          _qtype(args), args.num_bits, int(fp4)):
        return None
    v = value.contiguous()
    if v.data_ptr() % (8 * v.element_size()):
        return None  # a view that starts in the middle of a vector
    keep = []
    gs_ptr = _gscale_ptr(global_scale, keep)
    scale_dtype = _scale_dtype(args, v.dtype, fp4)
    zp_dtype = _zp_dtype(args)
    out = torch.empty_like(v)
    scales = zps = None
    if return_qparams:
        scales = torch.empty(out_shape, dtype=scale_dtype, device=v.device)
        zps = torch.empty(out_shape, dtype=zp_dtype, device=v.device)
    _lib.check(
        lib.ctmi_dynamic_qdq(
            v.data_ptr(), _lib.dtype_code(v.dtype), out.data_ptr(), rows, cols, blk_cols,
            _qtype(args), args.num_bits, int(args.symmetric), gs_ptr,
            scales.data_ptr() if return_qparams else None, _lib.dtype_code(scale_dtype),
            zps.data_ptr() if return_qparams else None, _lib.dtype_code(zp_dtype),
            _lib.stream_of(v.device),
        )
    )
    return (out, scales, zps) if return_qparams else out


def compute_dynamic_scales_and_zp(
    value: torch.Tensor,
    args: QuantizationArgs,
    module: Optional[torch.nn.Module] = None,
    global_scale: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Dynamic activation qparams (helpers.py:149-205).  TOKEN reduces every dim
    except 0 and 1 (so a 2-D input degenerates to one scale for the whole
    tensor, as in the reference); GROUP / TENSOR_GROUP reduce each run of
    group_size along the last dim; TENSOR reduces everything."""
    _lib.require_gpu(value)
    if value.dtype not in _FLOATS:
        raise NotImplementedError(f"cannot observe a tensor of dtype {value.dtype}")
    if not args.symmetric and is_fp4(args):
        raise NotImplementedError("Asymmetric Quantization is not supported for FP4")
    strategy = args.strategy
    if strategy == QuantizationStrategy.TOKEN.value:
        if value.ndim > 2:
            b, s = value.shape[0], value.shape[1]
            flat = value.reshape(b * s, -1)
            out_shape = (b, s) + (1,) * (value.ndim - 2)
            return _observe_rows(flat, flat.shape[-1], args, global_scale, out_shape)
        whole = True
    elif strategy == QuantizationStrategy.TENSOR.value:
        whole = True
    elif strategy in (QuantizationStrategy.TENSOR_GROUP.value, QuantizationStrategy.GROUP.value):
        g = args.group_size
        n_groups = math.ceil(value.shape[-1] / g)
        if n_groups * g != value.shape[-1]:
            raise RuntimeError(
                f"cannot split last dim {value.shape[-1]} into groups of {g}"
            )
        out_shape = tuple(value.shape[:-1]) + (n_groups,)
        return _observe_rows(value, g, args, global_scale, out_shape)
    else:
        supported = (
            QuantizationStrategy.TOKEN,
            QuantizationStrategy.TENSOR,
            QuantizationStrategy.TENSOR_GROUP,
            QuantizationStrategy.GROUP,
        )
        raise ValueError("Dynamic quantization is only supported for ", f"{supported}")
    assert whole
    cols = value.shape[-1] if value.ndim else 1
    rows = max(value.numel() // max(cols, 1), 1)
    mn, mx = minmax(value.reshape(rows, cols), rows, cols)
    # torch.aminmax yields 0-d tensors; calculate_qparams reshapes its 0-d results to [1]
    return calculate_qparams(mn.reshape(()), mx.reshape(()), args, global_scale=global_scale)


def observe_weight_qparams(
    weight: torch.Tensor,
    args: QuantizationArgs,
    global_scale: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Static min-max observer for a 2-D weight: amin/amax per tensor / channel /
    group / block (tests/mock_observer.py:38-113) followed by calculate_qparams,
    fused into one pass where the slice is one row tall.  Returns (scale,
    zero_point) with the shapes initialize_qparams expects
    (quantization/lifecycle/initialize.py:201-280)."""
    _lib.require_gpu(weight)
    if weight.ndim != 2:
        raise NotImplementedError("weight observers expect a 2-D tensor")
    rows, cols = weight.shape
    s = args.strategy
    if s == QuantizationStrategy.TENSOR.value:
        mn, mx = minmax(weight, rows, cols)
        return calculate_qparams(mn.reshape(1), mx.reshape(1), args, global_scale=global_scale)
    if s == QuantizationStrategy.CHANNEL.value:
        return _observe_rows(weight, cols, args, global_scale, (rows, 1))
    if s in (QuantizationStrategy.GROUP.value, QuantizationStrategy.TENSOR_GROUP.value):
        n_groups = strategy_cdiv(cols, args.group_size, s, strict=True)
        return _observe_rows(weight, args.group_size, args, global_scale, (rows, n_groups))
    if s == QuantizationStrategy.BLOCK.value:
        bh, bw = args.block_structure
        strategy_cdiv(rows, bh, s, strict=True)
        strategy_cdiv(cols, bw, s, strict=True)
        mn, mx = minmax(weight, bh, bw)
        return calculate_qparams(mn, mx, args, global_scale=global_scale)
    raise ValueError(f"{s} quantization cannot be applied to weights")


def observe_weights_qparams(weights, args: QuantizationArgs, global_scales=None):
    """observe_weight_qparams for a list of 2-D weights (a calibration pass over the modules
    of a model with the min-max observer, tests/mock_observer.py:38-113): channel and group
    strategies go to the GPU in one call (ctmi_observe_qparams_many, 8 weights per launch),
    the others one by one.  global_scales: one per weight or None.  Returns a list of
    (scale, zero_point)."""
    import ctypes

    import numpy as np

    n = len(weights)
    out = [None] * n
    s = args.strategy
    rowwise = s in (QuantizationStrategy.CHANNEL.value, QuantizationStrategy.GROUP.value,
                    QuantizationStrategy.TENSOR_GROUP.value)
    picked = []
    for i, w in enumerate(weights):
        gs = None if global_scales is None else global_scales[i]
        use_gs = gs is not None and is_fp4(args) and args.symmetric
        if (not rowwise or w.ndim != 2 or w.numel() == 0 or w.device.type != "cuda" or w.dtype not in _FLOATS
                or not w.is_contiguous()
                or (use_gs and (gs.device != w.device or gs.dtype is not torch.float32 or gs.numel() != 1))):
            out[i] = observe_weight_qparams(w, args, global_scale=gs)
            continue
        rows, cols = w.shape
        if s == QuantizationStrategy.CHANNEL.value:
            blk_cols, n_groups = cols, 1
        else:
            blk_cols, n_groups = args.group_size, strategy_cdiv(cols, args.group_size, s, strict=True)
        picked.append((i, w, gs if use_gs else None, blk_cols, (rows, n_groups)))
    if not picked:
        return out
    from compressed_tensors_amd.compressors.job_tables import slab_outputs

    zp_dtype = _zp_dtype(args)
    groups = {}
    for item in picked:
        i, w, gs, blk_cols, shape = item
        groups.setdefault((_scale_dtype(args, w.dtype, gs is not None), w.device), []).append(item)
    job_t = np.dtype(_lib.ObserveJob)
    for (scale_dtype, device), items in groups.items():
        scales = slab_outputs([it[4] for it in items], scale_dtype, device)
        zps = slab_outputs([it[4] for it in items], zp_dtype, device)
        tab = np.zeros(len(items), job_t)
        tab["x"] = [it[1].data_ptr() for it in items]
        tab["scale"] = [t.data_ptr() for t in scales]
        tab["zero_point"] = [t.data_ptr() for t in zps]
        tab["global_scale"] = [0 if it[2] is None else it[2].data_ptr() for it in items]
        tab["rows"] = [it[4][0] for it in items]
        tab["cols"] = [it[1].shape[1] for it in items]
        tab["blk_cols"] = [it[3] for it in items]
        tab["x_dtype"] = [_lib.dtype_code(it[1].dtype) for it in items]
        _lib.check(_lib.load().ctmi_observe_qparams_many(
            ctypes.cast(tab.ctypes.data, ctypes.POINTER(_lib.ObserveJob)), len(items), _qtype(args),
            args.num_bits, int(args.symmetric), -1, _lib.dtype_code(zp_dtype), _lib.stream_of(device)))
        for it, sc, zp in zip(items, scales, zps):
            out[it[0]] = (sc, zp)
    return out


def generate_gparam(
    updated_min_val: torch.Tensor,
    updated_max_val: torch.Tensor,
    scale_data=FP8_E4M3_DATA,
    quant_data=FP4_E2M1_DATA,
    dtype: Optional[torch.dtype] = torch.float32,
) -> torch.Tensor:
    """NVFP4 global scale = 448 * 6 / max|x| (helpers.py:414-434)."""
    if scale_data is not FP8_E4M3_DATA or quant_data is not FP4_E2M1_DATA:
        raise NotImplementedError("only fp8-e4m3 scales over fp4-e2m1 data are supported")
    _lib.require_gpu(updated_min_val, updated_max_val)
    mn = updated_min_val.contiguous()
    mx = updated_max_val.to(mn.dtype).contiguous()
    out = torch.empty(mn.shape, dtype=torch.float32, device=mn.device)
    _lib.check(
        _lib.load().ctmi_generate_gparam(mn.data_ptr(), mx.data_ptr(), _lib.dtype_code(mn.dtype),
                                         mn.numel(), out.data_ptr(), _lib.stream_of(mn.device))
    )
    return out.to(dtype).reshape([1])


def get_torch_bit_depth(value: torch.Tensor) -> int:
    try:
        return torch.finfo(value.dtype).bits
    except TypeError:
        return torch.iinfo(value.dtype).bits


def can_quantize(value: torch.Tensor, quant_args: QuantizationArgs) -> bool:
    """False when `value` already is as narrow as quant_args asks (helpers.py:373-390)."""
    bit_depth = get_torch_bit_depth(value)
    if bit_depth < quant_args.num_bits:
        _LOGGER.warning(
            f"Can't quantize tensor with bit depth {bit_depth} to {quant_args.num_bits}."
            "The QuantizationArgs provided are not compatible with the input tensor."
        )
    return bit_depth > quant_args.num_bits


def strategy_cdiv(value: int, divisor: int, strategy, strict: bool = False) -> int:
    dividend = math.ceil(value / divisor)
    if dividend * divisor != value:
        message = (
            f"{strategy} quantization strategy requires strict division of "
            f"weight/activation size {value} and group/block size {divisor}. "
            "consider reducing the group/block size or ignoring modules with "
            f"weights not divisible by {divisor}"
        )
        if strict:
            raise ValueError(message)
        _LOGGER.warning(message)
    return dividend
