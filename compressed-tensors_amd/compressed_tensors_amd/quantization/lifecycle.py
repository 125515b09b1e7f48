"""The steps around the kernels that put a quantization config on a model.

Names and behaviour follow the reference's quantization/lifecycle package:
  apply_quantization_config              apply.py:112-189
  load_pretrained_quantization_parameters apply.py:60-109
  compress_quantized_weights             compressed.py:33-73
  enable_quantization / disable_quantization   helpers.py:27-32
  is_module_quantized, is_model_quantized, module_type, iter_named_leaf_modules,
  iter_named_quantizable_modules         quantization/utils/helpers.py:237-330
Matching of targets is by module name, class name or `re:` expression
(utils/match.py:40-100); the first target of the config that matches a module decides
its scheme.
"""
from collections import OrderedDict
from copy import deepcopy
from typing import Generator, Optional, Tuple

import torch
from torch.nn import Module

from compressed_tensors_amd.config import CompressionFormat, QuantizationStatus
from compressed_tensors_amd.quantization.forward import quantize
from compressed_tensors_amd.quantization.initialize import (
    initialize_module_for_quantization,
    is_attention_module,
)
from compressed_tensors_amd.quantization.quant_scheme import QuantizationConfig, QuantizationScheme

__all__ = [
    "apply_quantization_config",
    "load_pretrained_quantization_parameters",
    "compress_quantized_weights",
    "enable_quantization",
    "disable_quantization",
    "is_module_quantized",
    "is_model_quantized",
    "module_type",
    "iter_named_leaf_modules",
    "iter_named_quantizable_modules",
]


def is_module_quantized(module: Module) -> bool:
    """does the module carry a scheme that quantizes anything?"""
    scheme = getattr(module, "quantization_scheme", None)
    return scheme is not None and any(
        a is not None for a in (scheme.weights, scheme.input_activations, scheme.output_activations))


def is_model_quantized(model: Module) -> bool:
    return any(is_module_quantized(m) for m in model.modules())


def module_type(module: Module) -> str:
    return type(module).__name__


def iter_named_leaf_modules(model: Module) -> Generator[Tuple[str, Module], None, None]:
    """modules without children (observers attached to a module do not make it a parent)"""
    for name, module in model.named_modules():
        children = [n for n, _ in module.named_children() if "observer" not in n]
        if not children and "observer" not in name:
            yield name, module


def iter_named_quantizable_modules(model: Module, include_children: bool = True,
                                   include_attn: bool = False,
                                   include_mlp: bool = False) -> Generator[Tuple[str, Module], None, None]:
    for name, module in model.named_modules():
        if include_children:
            children = [n for n, _ in module.named_children() if "observer" not in n]
            if not children and "observer" not in name:
                yield name, module
        if include_attn and name.endswith("self_attn"):
            yield name, module
        if include_mlp and name.endswith("mlp"):
            yield name, module


def enable_quantization(module: Module) -> None:
    module.quantization_enabled = True


def disable_quantization(module: Module) -> None:
    module.quantization_enabled = False


def apply_quantization_config(model: Module, config: Optional[QuantizationConfig],
                              run_compressed: bool = False):
    """attach the schemes of `config` to the modules they target and give these their
    scales and zero points (initialize_module_for_quantization); with run_compressed and a
    format other than dense a Linear becomes a CompressedLinear that holds the compressed
    parameters.  A kv_cache_scheme goes onto every attention module."""
    from compressed_tensors_amd.linear.compressed_linear import CompressedLinear
    from compressed_tensors_amd.modeling import initialize_hooked_attention, initialize_hooked_kv_cache

    config = deepcopy(config)
    if config is None:
        return dict()
    status = QuantizationStatus(getattr(config.quantization_status, "value", config.quantization_status))
    force_zero_point = status != QuantizationStatus.COMPRESSED
    if config.kv_cache_scheme is not None:
        kv_scheme = QuantizationScheme(targets=[".*self_attn$"], input_activations=config.kv_cache_scheme)
        for module in model.modules():
            if is_attention_module(module):
                module.quantization_scheme = kv_scheme
                initialize_hooked_kv_cache(model, module)
                initialize_module_for_quantization(module, force_zero_point=False)
                module.quantization_status = status
    target_to_scheme = OrderedDict()
    for scheme in config.config_groups.values():
        for target in scheme.targets:
            target_to_scheme[target] = scheme
    from compressed_tensors_amd.utils.match import is_narrow_match, match_named_modules, match_targets

    # a target that names no module is worth a warning; of several targets that name a module
    # the most specific decides: its name, then a pattern, then a class (apply.py:140-160)
    for name, module in list(match_named_modules(model, target_to_scheme, config.ignore, warn_on_fail=True)):
        scheme = target_to_scheme[match_targets(name, module, target_to_scheme)[0]]
        module.quantization_scheme = scheme
        if (run_compressed and isinstance(module, torch.nn.Linear)
                and config.format != CompressionFormat.dense.value):
            CompressedLinear.from_linear(module, quantization_scheme=scheme, quantization_format=config.format)
        else:
            if is_attention_module(module) and is_narrow_match(model, scheme.targets, name):
                initialize_hooked_attention(model, module)
            initialize_module_for_quantization(module, force_zero_point=force_zero_point)
        module.quantization_status = status


def load_pretrained_quantization_parameters(model: Module, model_name_or_path: Optional[str] = None,
                                            load_weight_qparams: Optional[bool] = False) -> None:
    """scales, zero points and g_idx of a compressed checkpoint into a model that
    apply_quantization_config has prepared: always those of inputs and outputs, those of the
    weights on request; a scale stored without a zero point gets zeros"""
    from compressed_tensors_amd.utils.safetensors_io import (
        CheckpointReader, get_quantization_parameter_to_path_mapping,
    )

    mapping = get_quantization_parameter_to_path_mapping(str(model_name_or_path))
    with CheckpointReader(str(model_name_or_path), device="cpu") as reader:
        for name, module in model.named_modules():
            if not is_module_quantized(module):
                continue
            scheme = module.quantization_scheme
            bases = [b for b, a in (("input", scheme.input_activations), ("output", scheme.output_activations))
                     if a is not None]
            if load_weight_qparams and scheme.weights is not None:
                bases.append("weight")
            for base in bases:
                g_idx = f"{name}.{base}_g_idx"
                if g_idx in mapping:
                    _set_data(module, f"{base}_g_idx", reader.get(g_idx))
                scale = f"{name}.{base}_scale"
                if scale not in mapping:
                    continue
                value = reader.get(scale)
                _set_data(module, f"{base}_scale", value)
                zp = f"{name}.{base}_zero_point"
                _set_data(module, f"{base}_zero_point", reader.get(zp) if zp in mapping else torch.zeros_like(value))


def _set_data(module: Module, name: str, value: torch.Tensor) -> None:
    param = getattr(module, name, None)
    if param is None:
        return
    if param.data.shape != value.shape:
        raise ValueError(f"{name}: stored shape {tuple(value.shape)} does not match {tuple(param.data.shape)}")
    param.data.copy_(value.to(device=param.data.device, dtype=param.data.dtype))


def compress_quantized_weights(module: Module) -> None:
    """the module's weight as int8 codes in place (`model.apply(compress_quantized_weights)`):
    quantize with the module's own scale, zero point and g_idx; a module without weight or
    scale is only marked compressed"""
    scheme = getattr(module, "quantization_scheme", None)
    if not scheme or not scheme.weights:
        return
    status = getattr(module, "quantization_status", None)
    if getattr(status, "value", status) == QuantizationStatus.COMPRESSED.value:
        return
    weight = getattr(module, "weight", None)
    scale = getattr(module, "weight_scale", None)
    if weight is None or scale is None:
        module.quantization_status = QuantizationStatus.COMPRESSED
        return
    module.weight.requires_grad = False  # no autograd through integer codes
    module.weight.data = quantize(
        x=weight.data, scale=scale.data, zero_point=getattr(module, "weight_zero_point", None),
        g_idx=getattr(module, "weight_g_idx", None), args=scheme.weights, dtype=torch.int8)
    module.quantization_status = QuantizationStatus.COMPRESSED
