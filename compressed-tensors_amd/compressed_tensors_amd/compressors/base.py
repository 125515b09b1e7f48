"""Abstract compressor: the plug-in interface every format implements.

Method names, arguments and return conventions follow the reference's
BaseCompressor (compressors/base.py:30-202).  Tensors are processed on the GPU
they live on; host tensors are first copied to the current GPU.
"""
from abc import ABC, abstractmethod
from typing import Dict, Generator, Optional, Tuple

import torch
from torch import Tensor
from torch.nn import Module

from compressed_tensors_amd.registry import RegistryMixin

__all__ = ["BaseCompressor", "to_gpu"]


def to_gpu(t: Optional[Tensor]) -> Optional[Tensor]:
    """Kernels only run on the GPU: move a host tensor to the current device."""
    if t is None or t.device.type == "cuda":
        return t
    if t.device.type == "meta":
        raise NotImplementedError("meta tensors carry no data to compress")
    if not torch.cuda.is_available():
        raise RuntimeError("compressed_tensors_amd needs a GPU (no CPU fallback exists)")
    return t.to(torch.device("cuda", torch.cuda.current_device()))


class BaseCompressor(RegistryMixin, ABC):
    def __init__(self, config=None):
        self.config = config

    def compression_param_info(self, weight_shape: torch.Size, quantization_args=None):
        raise NotImplementedError()

    @property
    @abstractmethod
    def compression_param_names(self) -> Tuple[str]:
        raise NotImplementedError()

    @abstractmethod
    def compress(self, model_state: Dict[str, Tensor], **kwargs) -> Dict[str, Tensor]:
        raise NotImplementedError()

    @abstractmethod
    def decompress(
        self, path_to_model_or_tensors, device: str = "cpu", **kwargs
    ) -> Generator[Tuple[str, Tensor], None, None]:
        raise NotImplementedError()

    def compress_weight(self, weight: Tensor, **kwargs) -> Dict[str, Tensor]:
        raise NotImplementedError()

    def decompress_weight(self, compressed_data: Dict[str, Tensor], **kwargs) -> Tensor:
        raise NotImplementedError()

    def compress_module(self, module: Module) -> Optional[Dict[str, Tensor]]:
        """Compress the weight of one quantized leaf module (base.py:125-151)."""
        scheme = getattr(module, "quantization_scheme", None)
        if scheme is None or not hasattr(scheme, "weights"):
            return None
        return self.compress_weight(
            weight=getattr(module, "weight", None),
            scale=getattr(module, "weight_scale", None),
            zero_point=getattr(module, "weight_zero_point", None),
            quantization_args=scheme.weights,
        )

    def decompress_module(self, module: Module):
        """Dense weight of one compressed leaf module (base.py:165-190)."""
        scheme = getattr(module, "quantization_scheme", None)
        if scheme is None or not hasattr(scheme, "weights"):
            return None
        device = next(module.parameters()).device
        compressed_data = {name: p for name, p in module.named_parameters()}
        return self.decompress_weight(
            compressed_data=compressed_data, quantization_args=scheme.weights
        ).to(device)
