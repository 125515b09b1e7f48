"""`naive-quantized` / `int-quantized` / `float-quantized`: weights stored in the
nearest torch dtype (int8 or float8_e4m3fn).

Reference: compressors/quantized_compressors/naive_quantized.py:36-154.
"""
from typing import Dict, Optional, Tuple

import torch
from torch import Tensor

from compressed_tensors_amd.compressors.base import BaseCompressor, to_gpu
from compressed_tensors_amd.compressors.quantized_base import BaseQuantizationCompressor
from compressed_tensors_amd.config import CompressionFormat
from compressed_tensors_amd.quantization.forward import dequantize, quantize
from compressed_tensors_amd.quantization.helpers import can_quantize
from compressed_tensors_amd.quantization.quant_args import QuantizationArgs

__all__ = [
    "NaiveQuantizationCompressor",
    "IntQuantizationCompressor",
    "FloatQuantizationCompressor",
]


@BaseCompressor.register(name=CompressionFormat.naive_quantized.value)
class NaiveQuantizationCompressor(BaseQuantizationCompressor):
    @property
    def compression_param_names(self) -> Tuple[str]:
        return ("weight", "weight_scale", "weight_zero_point", "weight_g_idx")

    def compression_param_info(
        self, weight_shape: torch.Size, quantization_args: Optional[QuantizationArgs] = None
    ) -> Dict[str, Tuple[torch.Size, torch.dtype]]:
        return {"weight": (weight_shape, quantization_args.pytorch_dtype())}

    def compress_weight(
        self,
        weight: Tensor,
        scale: Tensor,
        quantization_args: QuantizationArgs,
        zero_point: Optional[Tensor] = None,
        g_idx: Optional[Tensor] = None,
        device: Optional[torch.device] = None,
        global_scale: Optional[Tensor] = None,
    ) -> Dict[str, Tensor]:
        if global_scale is not None:
            raise ValueError("global_scale is not supported for the NaiveQuantizationCompressor")
        weight, scale, zero_point, g_idx = (to_gpu(t) for t in (weight, scale, zero_point, g_idx))
        if can_quantize(weight, quantization_args):
            quantized = quantize(
                x=weight,
                scale=scale,
                zero_point=zero_point,
                g_idx=g_idx,
                args=quantization_args,
                dtype=quantization_args.pytorch_dtype(),
            )
        else:
            quantized = weight
        if device is not None:
            quantized = quantized.to(device)
        return {"weight": quantized}

    def decompress_weight(
        self,
        compressed_data: Dict[str, Tensor],
        quantization_args: Optional[QuantizationArgs] = None,
    ) -> Tensor:
        return dequantize(
            x_q=to_gpu(compressed_data["weight"]),
            scale=to_gpu(compressed_data["weight_scale"]),
            zero_point=to_gpu(compressed_data.get("weight_zero_point", None)),
            g_idx=to_gpu(compressed_data.get("weight_g_idx", None)),
        )


@BaseCompressor.register(name=CompressionFormat.int_quantized.value)
class IntQuantizationCompressor(NaiveQuantizationCompressor):
    pass


@BaseCompressor.register(name=CompressionFormat.float_quantized.value)
class FloatQuantizationCompressor(NaiveQuantizationCompressor):
    pass
