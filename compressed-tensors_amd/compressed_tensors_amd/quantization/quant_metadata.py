"""Names of the quantization parameters a module may carry (reference:
src/compressed_tensors/quantization/quant_metadata.py)."""
from enum import Enum
from typing import List

from torch.nn import Module

__all__ = ["QuantizationMetadata", "KVCacheScaleType"]


class KVCacheScaleType(Enum):
    KEY = "k_scale"
    VALUE = "v_scale"


class QuantizationMetadata:
    @staticmethod
    def all_qparam_names() -> List[str]:
        """every parameter the quantization lifecycle may register on a module: the key /
        value cache scales and, for input, weight and output, the global scale, scale,
        zero point and g_idx (quant_metadata.py:34-50)"""
        return [KVCacheScaleType.KEY.value, KVCacheScaleType.VALUE.value] + [
            f"{base}_{suffix}" for base in ("input", "weight", "output")
            for suffix in ("global_scale", "scale", "zero_point", "g_idx")]

    @classmethod
    def clear_all_qparams(cls, module: Module) -> None:
        """take those a module holds off it again (quant_metadata.py:52-62)"""
        for name in cls.all_qparam_names():
            if hasattr(module, name):
                delattr(module, name)
