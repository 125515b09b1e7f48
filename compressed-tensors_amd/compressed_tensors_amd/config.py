"""Format names and the small config records the compressors consult.

Format strings are the registry keys of the reference
(config/base.py:26-60 CompressionFormat, SparsityStructure) and must not change:
they are what model configs on disk name.
"""
from enum import Enum, unique
from typing import Any, Dict, List, Optional

from compressed_tensors_amd.registry import RegistryMixin

__all__ = [
    "CompressionFormat",
    "SparsityStructure",
    "SparsityCompressionConfig",
    "DenseSparsityConfig",
    "BitmaskConfig",
    "Sparse24BitMaskConfig",
    "QuantizationStatus",
    "LIFECYCLE_ORDER",
    "DEFAULT_QUANTIZATION_METHOD",
    "DEFAULT_QUANTIZATION_FORMAT",
    "SPARSITY_CONFIG_NAME",
    "QUANTIZATION_CONFIG_NAME",
    "TRANSFORM_CONFIG_NAME",
    "COMPRESSION_VERSION_NAME",
    "QUANTIZATION_METHOD_NAME",
    "infer_and_set_per_module_quantization_format",
]

SPARSITY_CONFIG_NAME = "sparsity_config"
QUANTIZATION_CONFIG_NAME = "quantization_config"
TRANSFORM_CONFIG_NAME = "transform_config"
COMPRESSION_VERSION_NAME = "version"
QUANTIZATION_METHOD_NAME = "quant_method"


@unique
class CompressionFormat(Enum):
    dense = "dense"
    sparse_bitmask = "sparse-bitmask"
    sparse_24_bitmask = "sparse-24-bitmask"
    int_quantized = "int-quantized"
    float_quantized = "float-quantized"
    naive_quantized = "naive-quantized"
    pack_quantized = "pack-quantized"
    marlin_24 = "marlin-24"
    mixed_precision = "mixed-precision"
    nvfp4_pack_quantized = "nvfp4-pack-quantized"
    mxfp4_pack_quantized = "mxfp4-pack-quantized"


@unique
class SparsityStructure(Enum):
    TWO_FOUR = "2:4"
    ZERO_ZERO = "0:0"
    UNSTRUCTURED = "unstructured"

    def __new__(cls, value):
        obj = object.__new__(cls)
        obj._value_ = value.lower()
        return obj

    @classmethod
    def _missing_(cls, value):
        if value is None:
            return cls.UNSTRUCTURED
        for member in cls:
            if member.value == str(value).lower():
                return member
        raise ValueError(f"{value} is not a valid {cls.__name__}")


class QuantizationStatus(str, Enum):
    """where a quantized layer is in its life; statuses compare by that order, and any
    status is at or beyond None (quantization/quant_config.py:39-99)"""
    INITIALIZED = "initialized"
    CALIBRATION = "calibration"
    FROZEN = "frozen"
    COMPRESSED = "compressed"

    @classmethod
    def lifecycle_order(cls) -> List["QuantizationStatus"]:
        return list(cls)

    def _rank_against(self, other):
        if not isinstance(other, QuantizationStatus):
            raise NotImplementedError
        order = LIFECYCLE_ORDER
        return order.index(self), order.index(other)

    def __ge__(self, other):
        if other is None:
            return True
        a, b = self._rank_against(other)
        return a >= b

    def __gt__(self, other):
        if other is None:
            return True
        a, b = self._rank_against(other)
        return a > b

    def __lt__(self, other):
        if other is None:
            return False
        a, b = self._rank_against(other)
        return a < b

    def __le__(self, other):
        if other is None:
            return False
        a, b = self._rank_against(other)
        return a <= b


LIFECYCLE_ORDER = [QuantizationStatus.INITIALIZED, QuantizationStatus.CALIBRATION,
                   QuantizationStatus.FROZEN, QuantizationStatus.COMPRESSED]
DEFAULT_QUANTIZATION_METHOD = "compressed-tensors"
DEFAULT_QUANTIZATION_FORMAT = "fakequant"


class SparsityCompressionConfig(RegistryMixin):
    """format / targets / ignore / global_sparsity / sparsity_structure
    (reference: config/base.py:97-114); the configs of the formats register under the
    format's name."""

    def __init__(
        self,
        format: str,
        targets: Optional[List[str]] = None,
        ignore: Optional[List[str]] = None,
        global_sparsity: float = 0.0,
        sparsity_structure: Optional[str] = "unstructured",
    ):
        self.format = format.value if isinstance(format, CompressionFormat) else format
        self.targets = targets
        self.ignore = ignore
        self.global_sparsity = global_sparsity
        self.sparsity_structure = sparsity_structure

    def model_dump(self) -> Dict[str, Any]:
        return dict(self.__dict__)

    @classmethod
    def load_from_registry(cls, name, **kwargs) -> "SparsityCompressionConfig":
        """the config class registered for a sparsity format, built from the fields of a
        config.json entry (config/base.py:97-114; other keys of the entry are ignored, as
        the reference's models ignore them)"""
        fields = ("format", "targets", "ignore", "global_sparsity", "sparsity_structure")
        return cls.get_value_from_registry(name)(**{k: v for k, v in kwargs.items() if k in fields})

    def __eq__(self, other) -> bool:
        return isinstance(other, SparsityCompressionConfig) and self.model_dump() == other.model_dump()

    __hash__ = None


@SparsityCompressionConfig.register(name=CompressionFormat.dense.value)
class DenseSparsityConfig(SparsityCompressionConfig):
    """config/dense.py:26-43: sparse tensors stored as they are"""

    def __init__(self, format: str = CompressionFormat.dense.value, **kwargs):
        super().__init__(format=format, **kwargs)


@SparsityCompressionConfig.register(name=CompressionFormat.sparse_bitmask.value)
class BitmaskConfig(SparsityCompressionConfig):
    """config/sparse_bitmask.py:26-40"""

    def __init__(self, format: str = CompressionFormat.sparse_bitmask.value, **kwargs):
        super().__init__(format=format, **kwargs)


@SparsityCompressionConfig.register(name=CompressionFormat.sparse_24_bitmask.value)
class Sparse24BitMaskConfig(SparsityCompressionConfig):
    """config/sparse_24_bitmask.py:27-40: 2:4 by default"""

    def __init__(self, format: str = CompressionFormat.sparse_24_bitmask.value,
                 sparsity_structure: Optional[str] = SparsityStructure.TWO_FOUR.value, **kwargs):
        super().__init__(format=format, sparsity_structure=sparsity_structure, **kwargs)


def _quant_compression_format(input_args, weight_args, sparsity_structure=None) -> CompressionFormat:
    """the format a module's weight and input arguments ask for (config/format.py:32-84)"""
    two_four = SparsityStructure(sparsity_structure) == SparsityStructure.TWO_FOUR
    if weight_args.num_bits == 4 and weight_args.type == "float":
        return CompressionFormat.nvfp4_pack_quantized
    if input_args is None:  # weight only: W4A16, W8A16
        if not (weight_args.num_bits in (4, 8) and weight_args.type == "int"):
            return CompressionFormat.naive_quantized
        if two_four and weight_args.strategy in ("channel", "group"):
            return CompressionFormat.marlin_24
        return CompressionFormat.pack_quantized
    if weight_args.type == "float" and weight_args.num_bits == 8:
        return CompressionFormat.float_quantized
    if weight_args.type == "int":
        return CompressionFormat.int_quantized
    return CompressionFormat.naive_quantized


def infer_and_set_per_module_quantization_format(model, sparsity_structure: Optional[str] = None,
                                                 quantization_format: Optional[str] = None) -> Optional[List[str]]:
    """sets `quantization_scheme.format` of every quantized module (the global format if one
    is given, else the module's own, else the inferred one) and returns the distinct formats
    of the model, None if no module is quantized (config/format.py:87-159)"""
    import logging

    formats: List[str] = []
    for module in model.modules():
        scheme = getattr(module, "quantization_scheme", None)
        if scheme is None or not any(
                a is not None for a in (scheme.weights, scheme.input_activations, scheme.output_activations)):
            continue
        if scheme.weights is not None:
            inferred = _quant_compression_format(scheme.input_activations, scheme.weights, sparsity_structure).value
            if quantization_format is not None:
                if quantization_format != inferred:
                    logging.getLogger(__name__).warning(
                        "The provided format for the module does not match the inferred format. "
                        "Compression may fail ")
                scheme.format = quantization_format
            elif scheme.format is not None:
                if scheme.format != inferred:
                    logging.getLogger(__name__).warning(
                        "The provided format for the module does not match the inferred format. "
                        "Compression may fail ")
            else:
                scheme.format = inferred
        if scheme.format and scheme.format not in formats:
            formats.append(scheme.format)
    return formats or None
