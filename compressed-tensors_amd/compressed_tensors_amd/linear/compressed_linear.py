"""CompressedLinear: a Linear whose parameters are the compressed form of its
weight; the dense weight is rebuilt on the GPU the first time it is needed.

Behaviour follows linear/compressed_linear.py:33-109 of the reference: a module
converted with `from_linear` carries exactly the parameters named by its
compressor's `compression_param_info` (plus the scales / zero points of its
scheme), is marked COMPRESSED, and turns FROZEN once its first forward call has
decompressed the weight.  Parameters live on the module's own device: there is
no offloading layer here.
"""
import warnings

import torch
from torch import Tensor
from torch.nn import Linear, Parameter
from torch.nn import functional as F

from compressed_tensors_amd.compressors.base import BaseCompressor
from compressed_tensors_amd.config import QuantizationStatus
from compressed_tensors_amd.quantization.initialize import initialize_module_for_quantization
from compressed_tensors_amd.quantization.quant_scheme import QuantizationScheme

__all__ = ["CompressedLinear"]


def _frozen(data: Tensor) -> Parameter:
    return Parameter(data, requires_grad=False)


class CompressedLinear(Linear):
    def __init__(self, *args, **kwargs) -> None:
        warnings.warn(
            "a CompressedLinear built by its constructor holds a dense weight and no "
            "compressor; convert an existing Linear with CompressedLinear.from_linear()",
            UserWarning,
            stacklevel=2,
        )
        super().__init__(*args, **kwargs)

    @classmethod
    @torch.no_grad()
    def from_linear(cls, module: Linear, quantization_scheme: QuantizationScheme,
                    quantization_format: str) -> "CompressedLinear":
        """Convert `module` in place (the same object is returned): its dense weight
        is replaced by uninitialised parameters with the compressed format's names,
        shapes and dtypes, ready to be filled from a compressed checkpoint."""
        compressor = BaseCompressor.load_from_registry(quantization_format)
        dense_shape, device = module.weight.shape, module.weight.device

        module.__class__ = cls
        module.compressor = compressor
        initialize_module_for_quantization(module, quantization_scheme, force_zero_point=False)
        layout = compressor.compression_param_info(dense_shape, quantization_scheme.weights)
        module._swap_weight_for(layout, device)
        module.quantization_status = QuantizationStatus.COMPRESSED
        return module

    def _swap_weight_for(self, layout, device) -> None:
        """drop the dense weight (and anything the compressed layout redefines), then
        register one empty parameter per entry of the layout"""
        for stale in {"weight", *layout}:
            if stale in self._parameters:
                del self._parameters[stale]
        for name, (shape, dtype) in layout.items():
            self.register_parameter(name, _frozen(torch.empty(shape, dtype=dtype, device=device)))

    def _materialise_weight(self) -> None:
        self.register_parameter("weight", _frozen(self.compressor.decompress_module(self)))
        self.quantization_status = QuantizationStatus.FROZEN

    def forward(self, input: Tensor) -> Tensor:
        if self.quantization_status == QuantizationStatus.COMPRESSED:
            self._materialise_weight()
        return F.linear(input, self.weight, self.bias)
