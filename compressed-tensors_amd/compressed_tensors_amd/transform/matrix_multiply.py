"""Transforms by an explicit random matrix (reference:
src/compressed_tensors/transform/factory/matrix_multiply.py).  The product with the matrix
runs in ctmi_kron_matmul / ctmi_block_matmul where the matrix fits the kernel's tile
(apply_transform_weight decides)."""
from typing import Dict, Optional

import torch
from torch import Tensor
from torch.nn import Module, Parameter

from .hadamard import (TransformArgs, TransformBase, TransformFactory, TransformScheme,
                       _transform_size, apply_transform_weight)

__all__ = ["RandomMatrixFactory", "RandomMatrixTransform", "high_precision_invert"]


def high_precision_invert(weight: Tensor) -> Tensor:
    """matrix_multiply.py:112-113: the inverse computed in float64, in the matrix' dtype"""
    return torch.linalg.inv(weight.to(torch.float64)).to(weight.dtype)


class RandomMatrixTransform(TransformBase):
    """value -> value times `weight` at the location (matrix_multiply.py:77-109); `weight`
    already is the inverse if args.inverse"""

    def __init__(self, weight: Tensor, scheme: TransformScheme, args: TransformArgs,
                 module_type: type):
        super().__init__()
        self.weight = weight
        self.scheme = scheme
        self.args = args
        self.module_type = module_type

    def same_as(self):
        return (id(self.weight), self.args.location, self.module_type)

    def forward(self, value: Tensor) -> Tensor:
        w = self.weight.detach()
        return apply_transform_weight(w, value.to(dtype=w.dtype), self.args.location,
                                      self.module_type).to(value.dtype)

    def right_inverse(self, value: Tensor) -> Tensor:
        inverse = high_precision_invert(self.weight.detach())
        return apply_transform_weight(inverse, value.to(dtype=inverse.dtype), self.args.location,
                                      self.module_type).to(value.dtype)


@TransformFactory.register("random-matrix")
class RandomMatrixFactory(TransformFactory):
    """One uniform random matrix per size, drawn from the factory's generator, and its
    inverse where asked for (matrix_multiply.py:31-74)."""

    def __init__(self, name: str, scheme: TransformScheme, seed: Optional[int] = None):
        super().__init__(name, scheme, seed)
        self._weights: Dict[int, Parameter] = {}
        self._inverses: Dict[int, Parameter] = {}

    def _create_weight(self, size: int, device, precision: torch.dtype) -> Parameter:
        data = torch.rand((size, size), generator=self.generator, dtype=precision,
                          device=self.generator.device).to(device)
        return Parameter(data, requires_grad=self.scheme.requires_grad)

    def _create_inverse(self, weight: Parameter) -> Parameter:
        return Parameter(high_precision_invert(weight.data).contiguous(), requires_grad=False)

    def _transform_key(self, module: Module, args: TransformArgs):
        return (_transform_size(module, args.location, self.scheme.head_dim), type(module))

    def create_transform(self, module: Module, args: TransformArgs) -> RandomMatrixTransform:
        size = _transform_size(module, args.location, self.scheme.head_dim)
        own = next(module.parameters(recurse=False), None)
        device = own.device if own is not None else torch.device("cpu")
        precision = self.scheme.precision if args.is_online() else torch.float64
        # one matrix per size: precision and device of the first use stay (the reference's
        # cache is keyed by the size alone), so that a transform and its inverse at two
        # locations of different precision are the same matrix
        if size not in self._weights:
            self._weights[size] = self._create_weight(size, device, precision)
        weight = self._weights[size]
        if args.inverse:
            if id(weight) not in self._inverses:
                self._inverses[id(weight)] = self._create_inverse(weight)
            weight = self._inverses[id(weight)]
        return RandomMatrixTransform(weight, self.scheme, args, type(module))
