"""Shapes and dtypes of the quantization parameters a module is given (host logic,
no GPU): the table of the reference's
tests/test_quantization/lifecycle/test_initialize.py:101-250, restated."""
import math

import pytest
import torch
from torch.nn import Linear

from compressed_tensors_amd.quantization import (
    QuantizationArgs,
    QuantizationScheme,
    initialize_module_for_quantization,
)

CASES = [
    (dict(strategy="tensor"), None),
    (dict(strategy="channel"), None),
    (dict(strategy="group", group_size=2), None),
    (dict(strategy="group", group_size=2, actorder="group"), None),
    (dict(strategy="group", group_size=2, actorder="weight"), None),
    (dict(strategy="tensor_group", group_size=2, type="float", num_bits=4), None),
    (dict(strategy="tensor_group", group_size=2, type="float", num_bits=4),
     dict(strategy="tensor_group", group_size=2, type="float", num_bits=4, dynamic="local")),
    (dict(strategy="block", block_structure=[2, 4]), None),
    (dict(strategy="tensor", symmetric=False), dict(strategy="tensor")),
    (dict(strategy="channel", num_bits=8, type="float"), dict(strategy="token", dynamic=True, num_bits=8, type="float")),
]


@pytest.mark.parametrize("weights,inputs", CASES)
def test_initialize_quantization_parameters(weights, inputs):
    scheme = QuantizationScheme(targets=["*"], weights=weights, input_activations=inputs)
    layer = Linear(8, 6)
    initialize_module_for_quantization(layer, scheme)
    for which, base in (("input_activations", "input"), ("weights", "weight")):
        args = getattr(scheme, which)
        if args is None:
            continue
        if args.strategy == "tensor_group":
            gs = getattr(layer, f"{base}_global_scale")
            assert gs.dtype == torch.float32 and gs.numel() == 1
            if which == "weights":
                assert layer.weight_scale.dtype == torch.float8_e4m3fn
        else:
            assert not hasattr(layer, f"{base}_global_scale")
        if args.strategy == "tensor":
            shape = (1,)
        elif args.strategy == "channel":
            shape = (layer.weight.shape[0], 1)
        elif args.strategy in ("group", "tensor_group"):
            shape = (layer.weight.shape[0], math.ceil(layer.weight.shape[1] / args.group_size))
        elif args.strategy == "block":
            bh, bw = args.block_structure
            shape = (math.ceil(layer.weight.shape[0] / bh), math.ceil(layer.weight.shape[1] / bw))
        else:
            shape = None
        if not args.dynamic:
            assert getattr(layer, f"{base}_scale").shape == shape
            assert getattr(layer, f"{base}_zero_point").shape == shape
            assert getattr(layer, f"{base}_scale").dtype == (
                torch.float8_e4m3fn if args.strategy == "tensor_group" else layer.weight.dtype)
        else:
            assert not hasattr(layer, f"{base}_scale")
        if args.actorder == "group":
            g_idx = getattr(layer, f"{base}_g_idx")
            assert g_idx.shape == (layer.weight.shape[1],) and bool((g_idx == -1).all())
        else:
            assert not hasattr(layer, f"{base}_g_idx")


def test_no_zero_point_unless_needed_and_reinitialisation():
    layer = Linear(8, 6)
    scheme = QuantizationScheme(targets=["*"], weights=dict(strategy="channel"))
    initialize_module_for_quantization(layer, scheme, force_zero_point=False)
    assert hasattr(layer, "weight_scale") and not hasattr(layer, "weight_zero_point")
    asym = QuantizationScheme(targets=["*"], weights=dict(strategy="tensor", symmetric=False))
    initialize_module_for_quantization(layer, asym, force_zero_point=False)
    assert layer.weight_scale.shape == (1,) and layer.weight_zero_point.dtype == torch.int8
    with pytest.raises(ValueError, match="static token"):
        initialize_module_for_quantization(
            layer, QuantizationScheme(targets=["*"], weights=dict(strategy="token")))
