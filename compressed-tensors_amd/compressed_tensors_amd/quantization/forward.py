"""quantize / dequantize / fake_quantize on the GPU.

Same signatures and semantics as the reference's
quantization/lifecycle/forward.py:45-189 (strategy dispatch :193-353, dynamic
activation entry `forward_quantize` :414-451).  The reference materialises the
op chain div -> (+zp) -> clamp -> round -> cast (and its mirror image) as
separate torch ops; here the strategy is reduced to a scale-grid description
(`QParams`) and one HIP kernel replays the whole chain per element.
"""
import ctypes
import functools
import math
from typing import Optional, Tuple

import torch

from compressed_tensors_amd import _lib
from compressed_tensors_amd.quantization.quant_args import (
    DynamicType,
    QuantizationArgs,
    QuantizationStrategy,
    QuantizationType,
)

__all__ = [
    "quantize",
    "dequantize",
    "fake_quantize",
    "forward_quantize",
    "wrap_module_forward_quantized",
    "build_qparams",
]

_FLOATS = (torch.float32, torch.float16, torch.bfloat16)
_GROUPED = (QuantizationStrategy.GROUP.value, QuantizationStrategy.TENSOR_GROUP.value)


def _promote(a: torch.dtype, b: torch.dtype) -> torch.dtype:
    return a if a == b else torch.float32


def _rows_cols(x) -> Tuple[int, int]:
    cols = x.shape[-1] if x.ndim else 1
    rows = x.numel() // cols if cols else 0
    return rows, cols


def _leading_grid(x_shape, s_shape) -> Tuple[int, int]:
    """Map the broadcast of scale dims over x's leading dims to
    (s_rows, blk_rows): scale row of flattened x row r = (r // blk_rows) % s_rows."""
    return _leading_grid_of(tuple(x_shape), tuple(s_shape))


@functools.lru_cache(maxsize=4096)
def _leading_grid_of(x_shape: tuple, s_shape: tuple) -> Tuple[int, int]:
    lead = list(x_shape[:-1])
    s_lead = list(s_shape)
    if len(s_lead) > len(lead):
        extra = s_lead[: len(s_lead) - len(lead)]
        if any(d != 1 for d in extra):
            raise NotImplementedError(f"scale shape {tuple(s_shape)} outranks tensor {tuple(x_shape)}")
        s_lead = s_lead[len(s_lead) - len(lead):]
    s_lead = [1] * (len(lead) - len(s_lead)) + s_lead
    for d, s in zip(lead, s_lead):
        if s != 1 and s != d:
            raise RuntimeError(f"scale shape {tuple(s_shape)} does not broadcast to {tuple(x_shape)}")
    active = [i for i, (d, s) in enumerate(zip(lead, s_lead)) if s != 1]
    if not active:
        return 1, max(1, math.prod(lead))
    lo, hi = active[0], active[-1]
    for i in range(lo, hi + 1):
        if s_lead[i] == 1 and lead[i] != 1:
            raise NotImplementedError(
                f"scale shape {tuple(s_shape)} is not a contiguous run of tensor dims"
            )
    s_rows = math.prod(lead[lo : hi + 1])
    blk_rows = max(1, math.prod(lead[hi + 1 :]))
    return s_rows, blk_rows


def _column_groups(g_idx: Optional[torch.Tensor], group_size: int) -> Optional[torch.Tensor]:
    """act-order: the reference sorts columns by g_idx and cuts the sorted order
    into runs of group_size (forward.py:286-303, 329-331)."""
    if g_idx is None:
        return None
    cols = g_idx.numel()
    if cols >= 1 << 16:  # beyond the counting kernel: torch's sort, with a host read-back
        if bool((g_idx == -1).any()):
            return None
        position = torch.argsort(torch.argsort(g_idx, stable=True))
        return (position // group_size).to(torch.int32).contiguous()
    g = g_idx.reshape(-1).to(torch.int32).contiguous()
    out = torch.empty_like(g)
    _lib.check(_lib.load().ctmi_column_groups(g.data_ptr(), cols, group_size, out.data_ptr(),
                                              _lib.stream_of(g.device)))
    return out


class QPlan:
    """Everything a kernel launch needs, plus the tensors that must stay alive."""

    def __init__(self):
        self.qp = _lib.QParams()
        self.keep = []
        self.compute_dtype = None  # dtype of the quantize chain
        self.dequant_dtype = None  # dtype of the dequantize chain
        self.grouped = False


class _ShapeOnly:
    """stand-in for a tensor of which only shape and dtype matter"""

    def __init__(self, shape, dtype):
        self.shape = torch.Size(shape)
        self.dtype = dtype
        self.ndim = len(self.shape)

    def numel(self):
        return math.prod(self.shape)


def build_qparams(
    x,
    scale: torch.Tensor,
    zero_point: Optional[torch.Tensor],
    args: QuantizationArgs,
    g_idx: Optional[torch.Tensor] = None,
    global_scale: Optional[torch.Tensor] = None,
) -> QPlan:
    """Translate (tensor shape, scale shape, strategy) into the scale-grid
    description the kernels consume.  `x` is the tensor, or a _ShapeOnly."""
    plan = QPlan()
    qp = plan.qp
    dev = _lib.require_gpu(
        x if isinstance(x, torch.Tensor) else None, scale, zero_point, g_idx, global_scale
    )
    rows, cols = _rows_cols(x)
    strategy = args.strategy

    if scale.dtype == torch.float64 or x.dtype == torch.float64:
        raise NotImplementedError("float64 quantization is not supported by the HIP kernels")

    if strategy == QuantizationStrategy.BLOCK.value:
        if x.ndim != 2:
            raise NotImplementedError("block quantization expects a 2-D tensor")
        bh, bw = args.block_structure
        if rows % bh != 0:
            raise ValueError(
                f"Tensor height {rows} is not divisible by block_height {bh}."
                f" Block quantization requires exact division."
            )
        if cols % bw != 0:
            raise ValueError(
                f"Tensor width {cols} is not divisible by block_width {bw}. "
                f"Block quantization requires exact division."
            )
        if tuple(scale.shape) != (rows // bh, cols // bw):
            raise RuntimeError(f"block scale must have shape {(rows // bh, cols // bw)}")
        qp.s_rows, qp.s_cols, qp.blk_rows, qp.blk_cols = rows // bh, cols // bw, bh, bw
    elif strategy in _GROUPED:
        plan.grouped = True
        group_size = args.group_size
        while scale.ndim < 2:
            scale = scale.unsqueeze(1)
            zero_point = zero_point.unsqueeze(1) if zero_point is not None else None
        if cols >= group_size and cols % group_size != 0:
            raise ValueError(
                "tensor column shape must be divisble "
                f"by the given group_size {group_size} but got {cols}"
            )
        if cols % group_size != 0:
            raise RuntimeError(f"cannot split {cols} columns into groups of {group_size}")
        n_groups = cols // group_size
        if scale.shape[-1] != n_groups and scale.shape[-1] != 1:
            raise RuntimeError(
                f"scale has {scale.shape[-1]} groups, tensor has {n_groups} of size {group_size}"
            )
        s_rows, blk_rows = _leading_grid(x.shape, scale.shape[:-1])
        qp.s_rows, qp.blk_rows = s_rows, blk_rows
        if scale.shape[-1] == 1:
            qp.s_cols, qp.blk_cols = 1, max(cols, 1)
        else:
            qp.s_cols, qp.blk_cols = n_groups, group_size
            col_group = _column_groups(g_idx, group_size)
            if col_group is not None:
                plan.keep.append(col_group)
                qp.col_group = col_group.data_ptr()
    else:  # tensor, channel, token, attn_head: plain broadcasting
        if scale.numel() == 1:
            qp.s_rows, qp.s_cols, qp.blk_rows, qp.blk_cols = 1, 1, max(rows, 1), max(cols, 1)
        else:
            last = scale.shape[-1]
            if last not in (1, cols):
                raise RuntimeError(f"scale shape {tuple(scale.shape)} does not broadcast to x")
            s_rows, blk_rows = _leading_grid(x.shape, scale.shape[:-1])
            qp.s_rows, qp.blk_rows = s_rows, blk_rows
            if last == 1:
                qp.s_cols, qp.blk_cols = 1, max(cols, 1)
            else:
                qp.s_cols, qp.blk_cols = cols, 1

    if zero_point is not None and zero_point.numel() != scale.numel():
        raise RuntimeError("zero_point must have as many elements as scale")

    scale_c = scale.contiguous()
    plan.keep.append(scale_c)
    qp.scale = scale_c.data_ptr()
    qp.scale_dtype = _lib.dtype_code(scale.dtype)
    if zero_point is not None:
        zp_c = zero_point.contiguous()
        plan.keep.append(zp_c)
        qp.zero_point = zp_c.data_ptr()
        qp.zp_dtype = _lib.dtype_code(zero_point.dtype)
    if global_scale is not None:
        gs = global_scale.to(torch.float32).reshape(-1).contiguous()
        if gs.numel() != 1:
            raise NotImplementedError("global_scale must hold a single value")
        plan.keep.append(gs)
        qp.global_scale = gs.data_ptr()

    qp.qtype = _lib.QTYPE_INT if args.type == QuantizationType.INT.value else _lib.QTYPE_FLOAT
    qp.num_bits = args.num_bits

    eff_scale_dtype = torch.float32 if global_scale is not None else scale.dtype
    plan.dequant_dtype = eff_scale_dtype
    if x.dtype in _FLOATS:
        plan.compute_dtype = _promote(x.dtype, eff_scale_dtype)
    else:
        plan.compute_dtype = eff_scale_dtype
    del dev
    return plan


def _run(
    x: torch.Tensor,
    scale: torch.Tensor,
    zero_point: Optional[torch.Tensor],
    args: QuantizationArgs,
    do_quantize: bool,
    do_dequantize: bool,
    dtype: Optional[torch.dtype],
    g_idx: Optional[torch.Tensor],
    global_scale: Optional[torch.Tensor],
) -> torch.Tensor:
    if do_quantize and x.dtype not in _FLOATS:
        raise NotImplementedError(f"cannot quantize a tensor of dtype {x.dtype}")
    if (
        do_quantize
        and scale.ndim == 0
        and global_scale is None
        and scale.dtype != x.dtype
        and args.strategy not in _GROUPED
    ):
        # a 0-d operand does not take part in type promotion: torch casts it to
        # the tensor's dtype before dividing
        if do_dequantize:
            raise NotImplementedError(
                "fake_quantize with a 0-d scale of another dtype than the input"
            )
        scale = scale.to(x.dtype)
    plan = build_qparams(x, scale, zero_point, args, g_idx, global_scale)

    # output dtype rules of _process_quantization
    if plan.grouped:
        out_dtype = dtype if dtype is not None else x.dtype  # forward.py:266, 327
    elif do_dequantize:
        out_dtype = plan.dequant_dtype  # _dequantize is called without dtype
    else:
        out_dtype = dtype if dtype is not None else plan.compute_dtype

    xc = x.contiguous()
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    rows, cols = _rows_cols(xc)
    lib = _lib.load()
    _lib.check(
        lib.ctmi_qdq(
            xc.data_ptr(),
            _lib.dtype_code(x.dtype),
            out.data_ptr(),
            _lib.dtype_code(out_dtype),
            rows,
            cols,
            ctypes.byref(plan.qp),
            int(do_quantize),
            int(do_dequantize),
            _lib.stream_of(x.device),
        )
    )
    return out


@torch.no_grad()
def quantize(
    x: torch.Tensor,
    scale: torch.Tensor,
    zero_point: Optional[torch.Tensor],
    args: QuantizationArgs,
    dtype: Optional[torch.dtype] = None,
    g_idx: Optional[torch.Tensor] = None,
    global_scale: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """reference: forward.py:45-81"""
    return _run(x, scale, zero_point, args, True, False, dtype, g_idx, global_scale)


_inferred: dict = {}


def infer_dequant_args(x_q: torch.Tensor, scale: torch.Tensor) -> QuantizationArgs:
    """strategy inference of `dequantize(args=None)`, forward.py:107-138.  The result
    depends on the two shapes only and is read, never changed: one object per pair of
    shapes (a model has a handful of them and hundreds of weights)."""
    key = (tuple(x_q.shape), tuple(scale.shape))
    args = _inferred.get(key)
    if args is None:
        if len(_inferred) > 4096:
            _inferred.clear()
        args = _inferred[key] = _infer_dequant_args(x_q, scale)
    return args


def _infer_dequant_args(x_q, scale) -> QuantizationArgs:
    if scale.ndim in (0, 1):
        return QuantizationArgs(strategy=QuantizationStrategy.TENSOR)
    if scale.ndim == 2:
        if scale.shape[1] == 1:
            return QuantizationArgs(strategy=QuantizationStrategy.CHANNEL)
        if scale.shape[0] == 1 or scale.shape[0] == x_q.shape[0]:
            group_size = int(x_q.shape[1] / scale.shape[1])
            return QuantizationArgs(strategy=QuantizationStrategy.GROUP, group_size=group_size)
        rows, cols = x_q.shape[-2], x_q.shape[-1]
        return QuantizationArgs(
            strategy=QuantizationStrategy.BLOCK,
            block_structure=[rows // scale.shape[0], cols // scale.shape[1]],
        )
    raise ValueError(
        f"Could not infer a quantization strategy from scale with {scale.ndim} "
        "dimmensions. Expected 0 or 2 dimmensions."
    )


@torch.no_grad()
def dequantize(
    x_q: torch.Tensor,
    scale: torch.Tensor,
    zero_point: Optional[torch.Tensor] = None,
    args: Optional[QuantizationArgs] = None,
    dtype: Optional[torch.dtype] = None,
    g_idx: Optional[torch.Tensor] = None,
    global_scale: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """reference: forward.py:85-153"""
    if args is None:
        args = infer_dequant_args(x_q, scale)
    if dtype is None:
        dtype = scale.dtype
    return _run(x_q, scale, zero_point, args, False, True, dtype, g_idx, global_scale)


@torch.no_grad()
def fake_quantize(
    x: torch.Tensor,
    scale: torch.Tensor,
    zero_point: Optional[torch.Tensor],
    args: QuantizationArgs,
    g_idx: Optional[torch.Tensor] = None,
    global_scale: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """reference: forward.py:157-189"""
    return _run(x, scale, zero_point, args, True, True, None, g_idx, global_scale)


def forward_quantize(
    module: torch.nn.Module, value: torch.Tensor, base_name: str, args: QuantizationArgs
) -> torch.Tensor:
    """reference: forward.py:414-451.  Dynamic schemes take one pass over `value`
    (scales and fake-quantization in one kernel) where a fused kernel exists, else
    the fused min/max + qparams kernel followed by fake_quantize."""
    from compressed_tensors_amd.quantization.helpers import (
        compute_dynamic_scales_and_zp, dynamic_fake_quantize,
    )

    status = getattr(module, "quantization_status", None)
    if status is not None and str(getattr(status, "value", status)) == "compressed":
        if base_name == "weight":
            return value
    if value.numel() == 0:
        return value

    g_idx = getattr(module, "weight_g_idx", None)
    global_scale = getattr(module, f"{base_name}_global_scale", None)

    if args.dynamic in (True, DynamicType.LOCAL.value):
        if g_idx is None:
            fused = dynamic_fake_quantize(value, args, global_scale)
            if fused is not None:
                return fused
        scale, zero_point = compute_dynamic_scales_and_zp(
            value=value, args=args, module=module, global_scale=global_scale
        )
    else:
        scale = getattr(module, f"{base_name}_scale")
        zero_point = getattr(module, f"{base_name}_zero_point", None)

    return fake_quantize(
        x=value, scale=scale, zero_point=zero_point, args=args, g_idx=g_idx,
        global_scale=global_scale,
    )


def wrap_module_forward_quantized(module: torch.nn.Module, scheme) -> None:
    """replace `module.forward` by one that fake-quantizes what the scheme names around the
    original call (forward.py:355-412): the input, the weight (put back afterwards; not for
    a compressed module, whose weight already lies on the grid) and the output (left alone
    while a static output scheme is being calibrated).  `module.quantization_enabled = False`
    switches all of it off."""
    from functools import wraps

    original = module.forward.__func__ if hasattr(module.forward, "__func__") else module.forward.func
    # a module that is initialized again is wrapped once, around the forward it came with
    original = getattr(original, "_wraps_forward", original)

    @wraps(original)
    def wrapped_forward(self, *args, **kwargs):
        call = original.__get__(module, module.__class__)
        if not getattr(module, "quantization_enabled", True):
            return call(*args, **kwargs)
        status = getattr(module, "quantization_status", None)
        status = str(getattr(status, "value", status))
        compressed = status == "compressed"
        input_ = args[0]
        if scheme.input_activations is not None:
            input_ = forward_quantize(module, input_, "input", scheme.input_activations)
        # (a CompressedLinear's weight was decompressed from codes: it lies on the grid already,
        # and its zero points may still be in their packed form)
        swap_weight = scheme.weights is not None and not compressed and not hasattr(module, "compressor")
        if swap_weight:
            kept = self.weight.data
            self.weight.data = forward_quantize(module, self.weight.data, "weight", scheme.weights)
        try:
            output = call(input_, *args[1:], **kwargs)
        finally:
            if swap_weight:
                self.weight.data = kept
        if scheme.output_activations is not None:
            if status == "calibration" and not scheme.output_activations.dynamic:
                return output
            output = forward_quantize(module, output, "output", scheme.output_activations)
        return output

    wrapped_forward._wraps_forward = original
    setattr(module, "forward", wrapped_forward.__get__(module, module.__class__))

