"""Format names and the small config records the compressors consult.

Format strings are the registry keys of the reference
(config/base.py:26-60 CompressionFormat, SparsityStructure) and must not change:
they are what model configs on disk name.
"""
from enum import Enum, unique
from typing import Any, Dict, List, Optional

__all__ = [
    "CompressionFormat",
    "SparsityStructure",
    "SparsityCompressionConfig",
    "QuantizationStatus",
    "SPARSITY_CONFIG_NAME",
    "QUANTIZATION_CONFIG_NAME",
]

SPARSITY_CONFIG_NAME = "sparsity_config"
QUANTIZATION_CONFIG_NAME = "quantization_config"


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
    INITIALIZED = "initialized"
    CALIBRATION = "calibration"
    FROZEN = "frozen"
    COMPRESSED = "compressed"


class SparsityCompressionConfig:
    """format / targets / ignore / global_sparsity / sparsity_structure
    (reference: config/base.py:97-114)."""

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
