"""Scale / zero-point parameters of a module that is about to be quantized.

Reference: quantization/lifecycle/initialize.py (initialize_module_for_quantization
:62-150, initialize_qparams :153-280): shapes and dtypes of `<base>_scale`,
`<base>_zero_point`, `<base>_global_scale` and `weight_g_idx` per strategy.  The
parameters are created on the device the module's weight lives on; attention
modules (k / v cache scales, :282-330) are outside this package's path.
"""
from typing import Optional, Tuple

import torch
from torch.nn import Module, Parameter

from compressed_tensors_amd.config import QuantizationStatus
from compressed_tensors_amd.quantization.helpers import FP8_DTYPE, is_fp4, strategy_cdiv
from compressed_tensors_amd.quantization.quant_args import (
    ActivationOrdering,
    DynamicType,
    QuantizationArgs,
    QuantizationStrategy,
)
from compressed_tensors_amd.quantization.quant_scheme import QuantizationScheme

__all__ = ["initialize_module_for_quantization", "initialize_qparams", "clear_qparams",
           "is_attention_module", "initialize_attn_qparams"]

_QPARAM_SUFFIXES = ("_scale", "_zero_point", "_global_scale", "_g_idx")
_BASE_NAMES = ("input", "weight", "output", "q", "k", "v")


def clear_qparams(module: Module) -> None:
    """remove quantization parameters left by an earlier scheme (initialize.py:85)"""
    for base in _BASE_NAMES:
        for suffix in _QPARAM_SUFFIXES:
            name = base + suffix
            if name in module._parameters:
                delattr(module, name)


def _device_of(module: Module) -> torch.device:
    """where the module computes: its weight, else its first parameter or buffer (those of
    its children included), else the CPU"""
    if isinstance(getattr(module, "weight", None), torch.Tensor):
        return module.weight.device
    for t in module.parameters():
        return t.device
    for t in module.buffers():
        return t.device
    return torch.device("cpu")


def _register(module: Module, name: str, value: torch.Tensor) -> None:
    if hasattr(module, name):
        delattr(module, name)
    module.register_parameter(name, Parameter(value, requires_grad=False))


def initialize_qparams(
    module: Module,
    base_name: str,
    quantization_args: QuantizationArgs,
    observed_shape: Tuple[int, ...],
    observed_dtype: torch.dtype,
    force_zero_point: bool = True,
) -> None:
    """reference: initialize.py:153-280"""
    args = quantization_args
    strategy = args.strategy
    dynamic = args.dynamic
    device = _device_of(module)

    if dynamic is True:  # scales are computed on the fly: nothing to hold
        return
    if strategy == QuantizationStrategy.TENSOR_GROUP.value:
        _register(module, f"{base_name}_global_scale",
                  torch.empty(1, dtype=torch.float32, device=device))
    if dynamic == DynamicType.LOCAL.value:
        return

    if strategy == QuantizationStrategy.TENSOR.value:
        expected_shape = (1,)
    elif strategy == QuantizationStrategy.TOKEN.value:
        raise ValueError("Cannot perform static token quantization")
    elif strategy == QuantizationStrategy.CHANNEL.value:
        if len(observed_shape) < 2:
            raise ValueError("Channel quant requires at least 2 observed dimensions")
        expected_shape = (observed_shape[-2], 1)
    elif strategy in (QuantizationStrategy.GROUP.value, QuantizationStrategy.TENSOR_GROUP.value):
        assert args.group_size is not None
        if len(observed_shape) < 1:
            raise ValueError("Group quant requires at least 1 observed dimension")
        num_groups = strategy_cdiv(observed_shape[-1], args.group_size, strategy)
        expected_shape = (*observed_shape[:-1], num_groups)
        if ActivationOrdering.GROUP == args.actorder:  # or its other name, dynamic
            _register(module, f"{base_name}_g_idx",
                      torch.full((observed_shape[-1],), -1, device=device, dtype=torch.int))
    elif strategy == QuantizationStrategy.BLOCK.value:
        assert args.block_structure is not None
        if len(observed_shape) < 2:
            raise ValueError("Block quant requires at least 2 observed dimensions")
        rows = strategy_cdiv(observed_shape[-2], args.block_structure[-2], strategy)
        cols = strategy_cdiv(observed_shape[-1], args.block_structure[-1], strategy)
        expected_shape = (rows, cols)
    elif strategy == QuantizationStrategy.ATTN_HEAD.value:
        if len(observed_shape) < 3:
            raise ValueError("Attention quant requires at least 3 observed dimensions")
        expected_shape = (observed_shape[-3], 1, 1)
    else:
        raise AssertionError(f"Unknown strategy {strategy}")

    if is_fp4(args):
        scale_dtype = zp_dtype = FP8_DTYPE
    else:
        scale_dtype = observed_dtype
        if scale_dtype not in (torch.float16, torch.bfloat16, torch.float32, torch.float64):
            scale_dtype = torch.bfloat16
        zp_dtype = args.pytorch_dtype()

    _register(module, f"{base_name}_scale",
              torch.empty(expected_shape, dtype=scale_dtype, device=device))
    if force_zero_point or not args.symmetric:
        _register(module, f"{base_name}_zero_point",
                  torch.zeros(expected_shape, dtype=zp_dtype, device=device))


def initialize_module_for_quantization(
    module: Module,
    scheme: Optional[QuantizationScheme] = None,
    force_zero_point: bool = True,
) -> None:
    """reference: initialize.py:62-150 (linear-like modules)"""
    scheme = scheme or getattr(module, "quantization_scheme", None)
    if scheme is None:
        return
    clear_qparams(module)
    if is_attention_module(module):
        initialize_attn_qparams(module, scheme, force_zero_point)
        module.quantization_scheme = scheme
        module.quantization_status = QuantizationStatus.INITIALIZED
        return
    if not hasattr(module, "weight"):
        return  # a weight is needed to know shapes and dtypes
    weight = module.weight
    if scheme.input_activations is not None:
        initialize_qparams(module, "input", scheme.input_activations, weight.shape[-1:],
                           weight.dtype, force_zero_point)
    if scheme.weights is not None:
        initialize_qparams(module, "weight", scheme.weights, weight.shape, weight.dtype,
                           force_zero_point)
    if scheme.output_activations is not None:
        initialize_qparams(module, "output", scheme.output_activations, weight.shape[:-1],
                           weight.dtype, force_zero_point)
    # forward calls act on the scheme from here on (forward.py:355-412)
    from compressed_tensors_amd.quantization.forward import wrap_module_forward_quantized

    wrap_module_forward_quantized(module, scheme)
    module.quantization_scheme = scheme
    module.quantization_status = QuantizationStatus.INITIALIZED


def is_attention_module(module: Module) -> bool:
    """reference: initialize.py:147-152"""
    return "attention" in module.__class__.__name__.lower() and (
        hasattr(module, "k_proj") or hasattr(module, "v_proj") or hasattr(module, "qkv_proj"))


def initialize_attn_qparams(module: Module, scheme: QuantizationScheme, force_zero_point: bool) -> None:
    """`q_*` parameters if the module calls attention through a QuantizedAttentionImpl, `k_*`
    and `v_*` if it writes through a QuantizedKVCache; observed shapes are
    (heads, None, head_dim) (reference: initialize.py:283-337)"""
    from compressed_tensors_amd.modeling import IMPL_ATTR, KV_CACHE_ATTR
    from compressed_tensors_amd.utils.helpers import get_head_dim, get_num_attn_heads, get_num_kv_heads

    impl = getattr(module, IMPL_ATTR, None)
    kv_cache = getattr(module, KV_CACHE_ATTR, None)
    if impl is None and kv_cache is None:
        raise ValueError(
            f"Attention module has quantization scheme but no {IMPL_ATTR} or {KV_CACHE_ATTR} "
            "attributes. Please ensure that these attributes are initialized using "
            "`initialize_hooked_attention`.")
    if scheme.weights is not None:
        raise ValueError("Cannot apply weight quantization to attention. Instead, target the "
                         "(q|k|v)_proj submodule layers of attention")
    if scheme.input_activations is None:
        raise ValueError("Cannot apply attention quantization without specifying input activations")
    if scheme.output_activations is not None:
        raise ValueError("Cannot apply output quantization to attention")
    config = (kv_cache if kv_cache is not None else impl).config
    head_dim = get_head_dim(config)
    dtype = next(module.parameters()).dtype
    if impl is not None:
        initialize_qparams(module, "q", scheme.input_activations,
                           (get_num_attn_heads(config), None, head_dim), dtype, force_zero_point)
    if kv_cache is not None:
        kv_shape = (get_num_kv_heads(config), None, head_dim)
        initialize_qparams(module, "k", scheme.input_activations, kv_shape, dtype, force_zero_point)
        initialize_qparams(module, "v", scheme.input_activations, kv_shape, dtype, force_zero_point)
