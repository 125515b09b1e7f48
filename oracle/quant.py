"""Oracle: quantization parameter math and quantize / dequantize.

Follows quantization/utils/helpers.py:67-234, 414-434, quantization/quant_args.py:55-68,
384-408 and quantization/lifecycle/forward.py:45-353, 455-514 of the reference,
op by op, on CPU tensors.  `args` is any object with the QuantizationArgs
attributes (num_bits, type, symmetric, strategy, group_size, block_structure),
enum-valued ones given as their string values.
"""
import math
from typing import Optional, Tuple

import torch

FP8 = torch.float8_e4m3fn
FP8_MAX, FP8_MIN = 448.0, -448.0
FP4_MAX, FP4_MIN = 6.0, -6.0


def is_fp4(args) -> bool:
    return args.num_bits == 4 and args.type == "float"


def pytorch_dtype(args) -> torch.dtype:
    # quant_args.py:361-375
    if args.type == "float":
        if args.num_bits == 8:
            return FP8
        raise NotImplementedError("Only num_bits in (8) are supported")
    if args.num_bits <= 8:
        return torch.int8
    if args.num_bits <= 16:
        return torch.int16
    return torch.int32


def calculate_range(args) -> Tuple[torch.Tensor, torch.Tensor]:
    # helpers.py:208-234 — 0-d fp32 tensors
    if args.type == "int":
        span = 2**args.num_bits
        return torch.tensor(-span / 2), torch.tensor(span / 2 - 1)
    if args.type == "float":
        if args.num_bits == 8:
            return torch.tensor(FP8_MIN), torch.tensor(FP8_MAX)
        if args.num_bits == 4:
            return torch.tensor(FP4_MIN), torch.tensor(FP4_MAX)
        raise NotImplementedError("Range calculation only supported for 4 and 8 bits")
    raise ValueError(f"Invalid quantization type {args.type}")


def calculate_qparams(min_vals, max_vals, args, global_scale=None):
    # helpers.py:67-146
    min_vals = torch.min(min_vals, torch.zeros_like(min_vals))
    max_vals = torch.max(max_vals, torch.zeros_like(max_vals))
    bit_min, bit_max = calculate_range(args)
    bit_range = bit_max - bit_min
    zp_dtype = FP8 if is_fp4(args) else pytorch_dtype(args)

    if args.symmetric:
        max_val_pos = torch.max(torch.abs(min_vals), torch.abs(max_vals))
        if is_fp4(args) and global_scale is not None:
            scales = global_scale * (max_val_pos / FP4_MAX)
            scales = torch.clamp(scales, max=FP8_MAX, min=FP8_MIN)
            scales = scales.to(FP8)
        else:
            scales = max_val_pos / (float(bit_range) / 2)
        if scales.dtype == FP8:
            scales = torch.where(scales == 0, torch.tensor(0.125, dtype=FP8), scales)
        else:
            scales = torch.clamp(scales, min=torch.finfo(torch.float32).eps)
        zero_points = torch.zeros(scales.shape, dtype=min_vals.dtype)
    else:
        if is_fp4(args):
            raise NotImplementedError("Asymmetric Quantization is not supported for FP4")
        scales = (max_vals - min_vals) / float(bit_range)
        scales = torch.clamp(scales, min=torch.finfo(torch.float32).eps)
        zero_points = bit_min - (min_vals / scales)
        zero_points = torch.clamp(zero_points, bit_min, bit_max)

    if args.type == "int":
        zero_points = torch.round(zero_points)
    zero_points = zero_points.to(zp_dtype)
    if scales.ndim == 0:
        scales = scales.reshape(1)
        zero_points = zero_points.reshape(1)
    return scales, zero_points


def generate_gparam(min_val, max_val, dtype=torch.float32):
    # helpers.py:414-434
    min_vals = torch.min(min_val, torch.zeros_like(min_val))
    max_vals = torch.max(max_val, torch.zeros_like(max_val))
    max_val_pos = torch.max(torch.abs(min_vals), torch.abs(max_vals))
    return (FP8_MAX * FP4_MAX / max_val_pos).to(dtype).reshape([1])


def compute_dynamic_scales_and_zp(value, args, global_scale=None):
    # helpers.py:149-205
    keep_dims = True
    if args.strategy == "token":
        reduce_dims = tuple(i for i in range(value.ndim) if i not in (0, 1))
    elif args.strategy == "tensor":
        reduce_dims = None
    elif args.strategy in ("tensor_group", "group"):
        reduce_dims, keep_dims = -1, False
        value = value.unflatten(-1, (math.ceil(value.shape[-1] / args.group_size), args.group_size))
    else:
        raise ValueError("Dynamic quantization is only supported for token/tensor/group")
    if not reduce_dims:
        min_val, max_val = torch.aminmax(value)
    else:
        min_val = torch.amin(value, dim=reduce_dims, keepdims=keep_dims)
        max_val = torch.amax(value, dim=reduce_dims, keepdims=keep_dims)
    return calculate_qparams(min_val, max_val, args, global_scale=global_scale)


def observe_weight(weight, args, global_scale=None):
    """min-max observer of tests/mock_observer.py:38-113 for a 2-D weight: amin/amax
    over dims (0, -1) of the strategy-flattened view, then calculate_qparams."""
    s = args.strategy
    if s == "tensor":
        obs = weight.reshape((1, 1, -1))
    elif s == "channel":
        obs = weight.unsqueeze(-2).unsqueeze(0)
    elif s in ("group", "tensor_group"):
        obs = weight.unflatten(-1, (-1, args.group_size)).unsqueeze(0)
    elif s == "block":
        bh, bw = args.block_structure
        r, c = weight.shape
        obs = weight.reshape(r // bh, bh, c // bw, bw).transpose(1, 2).flatten(-2, -1).unsqueeze(0)
    else:
        raise ValueError(s)
    mn = torch.amin(obs, dim=(0, -1))
    mx = torch.amax(obs, dim=(0, -1))
    return calculate_qparams(mn, mx, args, global_scale=global_scale)


def cast_to_fp4(x):
    # quant_args.py:55-68 (the in-place bucket writes, in order)
    sign = torch.sign(x)
    x = torch.abs(x)
    x[(x >= 0.0) & (x <= 0.25)] = 0.0
    x[(x > 0.25) & (x < 0.75)] = 0.5
    x[(x >= 0.75) & (x <= 1.25)] = 1.0
    x[(x > 1.25) & (x < 1.75)] = 1.5
    x[(x >= 1.75) & (x <= 2.5)] = 2.0
    x[(x > 2.5) & (x < 3.5)] = 3.0
    x[(x >= 3.5) & (x <= 5.0)] = 4.0
    x[x > 5.0] = 6.0
    return x * sign


def round_to_quantized_type(tensor, args):
    # quant_args.py:384-408
    original = tensor.dtype
    if args.type == "float":
        if args.num_bits == 8:
            rounded = tensor.to(FP8)
        elif args.num_bits == 4:
            rounded = cast_to_fp4(tensor)
        else:
            raise NotImplementedError("Only num_bits in (4, 8) are supported")
    elif args.type == "int":
        rounded = torch.round(tensor)
    else:
        raise ValueError(f"Invalid quantization type {args.type}")
    return rounded.to(original)


def _quantize(x, scale, zero_point, q_min, q_max, args, dtype=None, global_scale=None):
    # forward.py:455-487
    if global_scale is not None:
        scale = scale.to(global_scale.dtype) / global_scale
    scaled = x / scale
    if zero_point is not None:
        scaled += zero_point.to(x.dtype)
    clamped = torch.clamp(scaled, q_min, q_max)
    q = round_to_quantized_type(clamped, args)
    if dtype is not None:
        q = q.to(dtype)
    return q


def _dequantize(x_q, scale, zero_point=None, dtype=None, global_scale=None):
    # forward.py:491-514
    if global_scale is not None:
        scale = scale.to(global_scale.dtype) / global_scale
    v = x_q.to(scale.dtype)
    if zero_point is not None:
        v = v - zero_point.to(scale.dtype)
    v = v * scale
    if dtype is not None:
        v = v.to(dtype)
    return v


def _process(x, scale, zero_point, args, g_idx=None, dtype=None, do_quantize=True,
             do_dequantize=True, global_scale=None):
    # forward.py:193-353
    q_min, q_max = calculate_range(args)
    group_size = args.group_size
    if args.strategy == "block":
        shape = x.shape
        rows, cols = x.shape[-2], x.shape[-1]
        bh, bw = args.block_structure
        if rows % bh != 0 or cols % bw != 0:
            raise ValueError("Block quantization requires exact division.")
        xb = x.reshape(rows // bh, bh, cols // bw, bw).transpose(1, 2)
        sb = scale.unsqueeze(-1).unsqueeze(-1)
        zb = zero_point.unsqueeze(-1).unsqueeze(-1) if zero_point is not None else None
        if do_quantize:
            xb = _quantize(xb, sb, zb, q_min, q_max, args, dtype=dtype, global_scale=global_scale)
        if do_dequantize:
            xb = _dequantize(xb, sb, zb, global_scale=global_scale)
        return xb.transpose(1, 2).reshape(shape)
    if args.strategy in ("group", "tensor_group"):
        output_dtype = dtype if dtype is not None else x.dtype
        output = torch.zeros_like(x).to(output_dtype)
        columns = output.shape[-1]
        while scale.ndim < 2:
            scale = scale.unsqueeze(1)
            zero_point = zero_point.unsqueeze(1) if zero_point is not None else None
        if columns >= group_size and columns % group_size != 0:
            raise ValueError("tensor column shape must be divisble by the given group_size")
        is_column_order = g_idx is None or -1 in g_idx
        if not is_column_order:
            perm = torch.argsort(g_idx)
            x = x.index_select(-1, perm)
        x = x.unflatten(-1, (math.ceil(x.shape[-1] / group_size), group_size))
        if do_quantize:
            output = _quantize(
                x, scale.unsqueeze(-1),
                zero_point.unsqueeze(-1) if zero_point is not None else None,
                q_min, q_max, args, dtype=dtype, global_scale=global_scale)
        if do_dequantize:
            src = output if do_quantize else x
            output = _dequantize(
                src, scale.unsqueeze(-1),
                zero_point.unsqueeze(-1) if zero_point is not None else None,
                global_scale=global_scale)
        output = output.flatten(start_dim=-2).to(output_dtype)
        if not is_column_order:
            output = output.index_select(-1, torch.argsort(perm))
        return output
    # tensor, channel, token, attn_head
    if do_quantize:
        output = _quantize(x, scale, zero_point, q_min, q_max, args, dtype=dtype,
                           global_scale=global_scale)
    if do_dequantize:
        output = _dequantize(output if do_quantize else x, scale, zero_point,
                             global_scale=global_scale)
    return output


class _Args:
    def __init__(self, **kw):
        self.num_bits = kw.get("num_bits", 8)
        self.type = kw.get("type", "int")
        self.symmetric = kw.get("symmetric", True)
        self.strategy = kw.get("strategy", "tensor")
        self.group_size = kw.get("group_size", None)
        self.block_structure = kw.get("block_structure", None)


def infer_args(x_q, scale):
    # forward.py:107-138
    if scale.ndim in (0, 1):
        return _Args(strategy="tensor")
    if scale.ndim == 2:
        if scale.shape[1] == 1:
            return _Args(strategy="channel")
        if scale.shape[0] == 1 or scale.shape[0] == x_q.shape[0]:
            return _Args(strategy="group", group_size=int(x_q.shape[1] / scale.shape[1]))
        rows, cols = x_q.shape[-2], x_q.shape[-1]
        return _Args(strategy="block",
                     block_structure=[rows // scale.shape[0], cols // scale.shape[1]])
    raise ValueError("Could not infer a quantization strategy")


@torch.no_grad()
def quantize(x, scale, zero_point, args, dtype=None, g_idx=None, global_scale=None):
    return _process(x, scale, zero_point, args, g_idx=g_idx, dtype=dtype, do_quantize=True,
                    do_dequantize=False, global_scale=global_scale)


@torch.no_grad()
def dequantize(x_q, scale, zero_point=None, args=None, dtype=None, g_idx=None, global_scale=None):
    if args is None:
        args = infer_args(x_q, scale)
    if dtype is None:
        dtype = scale.dtype
    return _process(x_q, scale, zero_point, args, g_idx=g_idx, dtype=dtype, do_quantize=False,
                    do_dequantize=True, global_scale=global_scale)


@torch.no_grad()
def fake_quantize(x, scale, zero_point, args, g_idx=None, global_scale=None):
    return _process(x, scale, zero_point, args, g_idx=g_idx, do_quantize=True,
                    do_dequantize=True, global_scale=global_scale)
