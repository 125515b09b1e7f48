"""CompressedLinear: a Linear that holds its weight in a compressed format and
decompresses it on the GPU at its first forward call.

Reference: linear/compressed_linear.py:33-109 (from_linear :48-93, forward :95-109).
"""
import warnings
from typing import Dict, Tuple

import torch
from torch import Tensor
from torch.nn import Parameter
from torch.nn.functional import linear
from torch.nn.modules import Linear

from compressed_tensors_amd.compressors.base import BaseCompressor
from compressed_tensors_amd.config import QuantizationStatus
from compressed_tensors_amd.quantization.initialize import initialize_module_for_quantization
from compressed_tensors_amd.quantization.quant_scheme import QuantizationScheme

__all__ = ["CompressedLinear"]


class CompressedLinear(Linear):
    def __init__(self, *args, **kwargs) -> None:
        super().__init__(*args, **kwargs)
        warnings.warn(
            "CompressedLinear should not be initialized directly. "
            "Use the from_linear method instead.",
            UserWarning,
        )

    @classmethod
    @torch.no_grad()
    def from_linear(cls, module: Linear, quantization_scheme: QuantizationScheme,
                    quantization_format: str):
        """turn a dense Linear into one that holds empty compressed parameters of the
        right shapes and dtypes, to be filled from a compressed checkpoint"""
        module.__class__ = CompressedLinear
        module.compressor = BaseCompressor.load_from_registry(quantization_format)
        init_device = module.weight.device

        # scales and zero points
        initialize_module_for_quantization(module, quantization_scheme, force_zero_point=False)

        compression_params: Dict[str, Tuple] = module.compressor.compression_param_info(
            module.weight.shape, quantization_scheme.weights
        )
        delattr(module, "weight")
        for name, (shape, dtype) in compression_params.items():
            if hasattr(module, name):
                delattr(module, name)
            module.register_parameter(
                name,
                Parameter(torch.empty(shape, device=init_device, dtype=dtype), requires_grad=False),
            )
        module.quantization_status = QuantizationStatus.COMPRESSED
        if hasattr(module, "_old_forward"):  # forward wrapped by accelerate hooks
            module._old_forward = CompressedLinear.forward.__get__(module, CompressedLinear)
        return module

    def forward(self, input: Tensor) -> Tensor:
        """decompress the weight (once), then the wrapped linear"""
        if self.quantization_status == QuantizationStatus.COMPRESSED:
            weight_data = self.compressor.decompress_module(self)
            self.register_parameter("weight", Parameter(weight_data, requires_grad=False))
            self.quantization_status = QuantizationStatus.FROZEN
        return linear(input, self.weight, self.bias)
