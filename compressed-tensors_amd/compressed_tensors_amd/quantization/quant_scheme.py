"""QuantizationScheme and the preset table (W4A16, FP8_DYNAMIC, NVFP4, ...).

Field names and preset contents follow the reference's
quantization/quant_scheme.py:36-339 so that scheme names used in recipes map
to the same arguments.
"""
from copy import deepcopy
from typing import Any, Dict, List, Optional

from compressed_tensors_amd.quantization.quant_args import (
    DynamicType,
    QuantizationArgs,
    QuantizationStrategy,
    QuantizationType,
)

__all__ = [
    "QuantizationScheme",
    "QuantizationConfig",
    "preset_name_to_scheme",
    "is_preset_scheme",
    "PRESET_SCHEMES",
]


class QuantizationScheme:
    def __init__(
        self,
        targets: List[str],
        weights: Optional[QuantizationArgs] = None,
        input_activations: Optional[QuantizationArgs] = None,
        output_activations: Optional[QuantizationArgs] = None,
        format: Optional[str] = None,
    ):
        self.targets = list(targets)
        self.weights = QuantizationArgs.model_validate(weights) if weights is not None else None
        self.input_activations = (
            QuantizationArgs.model_validate(input_activations)
            if input_activations is not None
            else None
        )
        self.output_activations = (
            QuantizationArgs.model_validate(output_activations)
            if output_activations is not None
            else None
        )
        self.format = format
        for args in (self.input_activations, self.output_activations):
            if args is not None and args.actorder is not None:
                raise ValueError("Cannot apply actorder to activations")

    def __eq__(self, other) -> bool:
        return isinstance(other, QuantizationScheme) and self.model_dump() == other.model_dump()

    __hash__ = None

    def model_dump(self) -> Dict[str, Any]:
        return {
            "targets": self.targets,
            "weights": self.weights.model_dump() if self.weights else None,
            "input_activations": self.input_activations.model_dump()
            if self.input_activations
            else None,
            "output_activations": self.output_activations.model_dump()
            if self.output_activations
            else None,
            "format": self.format,
        }


class QuantizationConfig:
    """config_groups / format / quantization_status / ignore
    (reference: quantization/quant_config.py:105-283, fields only)."""

    def __init__(
        self,
        config_groups: Dict[str, QuantizationScheme],
        format: str = "fakequant",
        quantization_status: str = "initialized",
        global_compression_ratio: Optional[float] = None,
        ignore: Optional[List[str]] = None,
        kv_cache_scheme: Optional[QuantizationArgs] = None,
        quant_method: str = "compressed-tensors",
    ):
        groups = {}
        for name, scheme in config_groups.items():
            if isinstance(scheme, dict):
                scheme = QuantizationScheme(**scheme)
            elif not isinstance(scheme, QuantizationScheme):
                # a list of targets under the name of a preset scheme (quant_config.py:148-160)
                scheme = preset_name_to_scheme(name=name, targets=list(scheme))
            groups[name] = scheme
        self.config_groups = groups
        self.format = format
        self.quantization_status = quantization_status
        self.global_compression_ratio = global_compression_ratio
        self.ignore = ignore or []
        if isinstance(kv_cache_scheme, dict):
            kv_cache_scheme = QuantizationArgs(**kv_cache_scheme)
        self.kv_cache_scheme = kv_cache_scheme
        self.quant_method = quant_method

    def to_dict(self) -> Dict[str, Any]:
        """model_dump under the name transformers' quantizer calls (quant_config.py:162-164)"""
        return self.model_dump()

    def requires_calibration_data(self) -> bool:
        """are there scales only data can give: a kv cache scheme, static or locally dynamic
        input activations, static output activations (quant_config.py:262-278)"""
        if self.kv_cache_scheme is not None:
            return True
        for scheme in self.config_groups.values():
            inputs, outputs = scheme.input_activations, scheme.output_activations
            if inputs is not None and inputs.dynamic in (False, DynamicType.LOCAL, DynamicType.LOCAL.value):
                return True
            if outputs is not None and not outputs.dynamic:
                return True
        return False

    def __eq__(self, other) -> bool:
        return isinstance(other, QuantizationConfig) and self.model_dump() == other.model_dump()

    __hash__ = None

    @classmethod
    def model_validate(cls, data) -> "QuantizationConfig":
        """a config from its plain-dict form (fields this class does not have are dropped)"""
        if isinstance(data, QuantizationConfig):
            return data
        fields = ("config_groups", "format", "quantization_status", "global_compression_ratio", "ignore",
                  "kv_cache_scheme", "quant_method")
        return cls(**{k: v for k, v in dict(data).items() if k in fields})

    @staticmethod
    def from_pretrained(model, format=None) -> Optional["QuantizationConfig"]:
        """the config of a model whose modules carry `quantization_scheme`
        (quantization/quant_config.py:166-260): one group per distinct scheme, modules of a
        quantized class without a scheme on the ignore list, the status of the last quantized
        module; None if nothing is quantized.  format: a format, a list of formats
        ("mixed-precision" if more than one) or None (int-quantized for a compressed model,
        dense otherwise)."""
        from compressed_tensors_amd.config import CompressionFormat, QuantizationStatus
        from compressed_tensors_amd.modeling import IMPL_ATTR
        from compressed_tensors_amd.quantization.initialize import is_attention_module

        def quantized(module) -> bool:
            scheme = getattr(module, "quantization_scheme", None)
            return scheme is not None and any(
                a is not None for a in (scheme.weights, scheme.input_activations, scheme.output_activations))

        schemes: List[QuantizationScheme] = []
        status = None
        quantized_types = set()
        unquantized: Dict[str, List[str]] = {}
        kv_cache_scheme = None
        for name, module in model.named_modules():
            layer_type = type(module).__name__
            attention = is_attention_module(module)
            has_group = quantized(module) and (not attention or hasattr(module, IMPL_ATTR))
            if has_group:
                status = getattr(module, "quantization_status", status)
                quantized_types.add(layer_type)
                if module.quantization_scheme not in schemes:
                    schemes.append(module.quantization_scheme)
            if quantized(module) and attention:
                status = getattr(module, "quantization_status", status)
                kv_cache_scheme = module.quantization_scheme.input_activations
            if not has_group:
                unquantized.setdefault(layer_type, []).append(name)
        if not schemes and kv_cache_scheme is None:
            return None
        ignore = [n for layer_type, names in unquantized.items() if layer_type in quantized_types for n in names]
        if format is None:
            compressed = getattr(status, "value", status) == QuantizationStatus.COMPRESSED.value
            format = (CompressionFormat.int_quantized if compressed else CompressionFormat.dense).value
        elif isinstance(format, (list, tuple)):
            format = CompressionFormat.mixed_precision.value if len(format) > 1 else format[0]
        return QuantizationConfig(
            config_groups={f"group_{i}": scheme for i, scheme in enumerate(schemes)},
            quantization_status=status, kv_cache_scheme=kv_cache_scheme,
            global_compression_ratio=None, format=format, ignore=ignore)

    def model_dump(self, exclude=None) -> Dict[str, Any]:
        """plain-dict form, as written into a model's config.json"""
        data = {
            "config_groups": {name: scheme.model_dump() for name, scheme in self.config_groups.items()},
            "format": self.format,
            "quantization_status": getattr(self.quantization_status, "value", self.quantization_status),
            "global_compression_ratio": self.global_compression_ratio,
            "ignore": list(self.ignore),
            "kv_cache_scheme": self.kv_cache_scheme.model_dump() if self.kv_cache_scheme else None,
            "quant_method": self.quant_method,
        }
        for key in exclude or ():
            data.pop(key, None)
        return data


def _w(**kw) -> Dict[str, QuantizationArgs]:
    return {"weights": QuantizationArgs(**kw)}


_INT8_W_CHANNEL = dict(num_bits=8, type=QuantizationType.INT, strategy=QuantizationStrategy.CHANNEL,
                       symmetric=True, dynamic=False)
_FP8_W_TENSOR = dict(num_bits=8, type=QuantizationType.FLOAT, strategy=QuantizationStrategy.TENSOR,
                     symmetric=True, dynamic=False)

PRESET_SCHEMES: Dict[str, Dict[str, QuantizationArgs]] = {
    "UNQUANTIZED": {},
    "W8A16": _w(**_INT8_W_CHANNEL),
    "W4A16": _w(num_bits=4, type=QuantizationType.INT, strategy=QuantizationStrategy.GROUP,
                group_size=128, symmetric=True, dynamic=False),
    "W4A16_ASYM": _w(num_bits=4, type=QuantizationType.INT, strategy=QuantizationStrategy.GROUP,
                     group_size=128, symmetric=False, dynamic=False),
    "W8A8": {
        "weights": QuantizationArgs(**_INT8_W_CHANNEL),
        "input_activations": QuantizationArgs(
            num_bits=8, type=QuantizationType.INT, strategy=QuantizationStrategy.TOKEN,
            symmetric=True, dynamic=True, observer=None),
    },
    "W4A8": {
        "weights": QuantizationArgs(num_bits=4, type=QuantizationType.INT,
                                    strategy=QuantizationStrategy.GROUP, group_size=128,
                                    symmetric=True, dynamic=False),
        "input_activations": QuantizationArgs(
            num_bits=8, type=QuantizationType.INT, strategy=QuantizationStrategy.TOKEN,
            symmetric=True, dynamic=True, observer=None),
    },
    "FP8": {
        "weights": QuantizationArgs(**_FP8_W_TENSOR),
        "input_activations": QuantizationArgs(**_FP8_W_TENSOR),
    },
    "FP8_DYNAMIC": {
        "weights": QuantizationArgs(num_bits=8, type=QuantizationType.FLOAT,
                                    strategy=QuantizationStrategy.CHANNEL, symmetric=True,
                                    dynamic=False),
        "input_activations": QuantizationArgs(
            num_bits=8, type=QuantizationType.FLOAT, strategy=QuantizationStrategy.TOKEN,
            symmetric=True, dynamic=True, observer=None),
    },
    "FP8_BLOCK": {
        "weights": QuantizationArgs(num_bits=8, type=QuantizationType.FLOAT,
                                    strategy=QuantizationStrategy.BLOCK, symmetric=True,
                                    dynamic=False, block_structure=[128, 128]),
        "input_activations": QuantizationArgs(
            num_bits=8, type=QuantizationType.FLOAT, strategy=QuantizationStrategy.GROUP,
            symmetric=True, dynamic=True, observer=None, group_size=128),
    },
    "NVFP4A16": _w(num_bits=4, type=QuantizationType.FLOAT,
                   strategy=QuantizationStrategy.TENSOR_GROUP, symmetric=True, dynamic=False,
                   group_size=16),
    "NVFP4": {
        "weights": QuantizationArgs(num_bits=4, type=QuantizationType.FLOAT,
                                    strategy=QuantizationStrategy.TENSOR_GROUP, symmetric=True,
                                    dynamic=False, group_size=16),
        "input_activations": QuantizationArgs(
            num_bits=4, type=QuantizationType.FLOAT, strategy=QuantizationStrategy.TENSOR_GROUP,
            symmetric=True, dynamic=DynamicType.LOCAL, group_size=16),
    },
}
PRESET_SCHEMES["INT8"] = PRESET_SCHEMES["W8A8"]


def preset_name_to_scheme(name: str, targets: List[str]) -> QuantizationScheme:
    name = name.upper()
    if name not in PRESET_SCHEMES:
        raise KeyError(
            f"Unknown preset scheme name {name}, available names: {list(PRESET_SCHEMES.keys())}"
        )
    return QuantizationScheme(targets=targets, **deepcopy(PRESET_SCHEMES[name]))


def is_preset_scheme(name: str) -> bool:
    return name.upper() in PRESET_SCHEMES
