"""Small host-side utilities under the reference's names (reference:
src/compressed_tensors/utils/helpers.py, tests/test_utils/test_helpers.py,
tests/test_quantization/test_quant_args.py::test_actorder)."""
import warnings
from types import SimpleNamespace

import pytest
import torch

from compressed_tensors_amd.quantization import ActivationOrdering, QuantizationArgs
from compressed_tensors_amd.utils import (ParameterizedDefaultDict, deprecated, fix_fsdp_module_name,
                                          is_compressed_tensors_config, patch_attr, replace_module)


def test_actorder_aliases():
    A = ActivationOrdering
    assert A.DYNAMIC == A.GROUP and A.STATIC == A.WEIGHT and A.GROUP != A.WEIGHT and A.DYNAMIC != A.STATIC
    assert A.GROUP == "dynamic" and "static" == A.WEIGHT and A.GROUP != "weight"
    assert len({A.GROUP, A.DYNAMIC, A.WEIGHT, A.STATIC}) == 2
    # test_quant_args.py:83-116
    assert QuantizationArgs(group_size=128, actorder=A.GROUP).strategy == "group"
    args = QuantizationArgs(group_size=128, actorder=A.DYNAMIC)
    assert args.strategy == "group" and args.actorder == A.GROUP and args.actorder == "dynamic"
    for order in ("group", "weight", "static"):
        with pytest.raises(ValueError):
            QuantizationArgs(group_size=None, actorder=order)
        with pytest.raises(ValueError):
            QuantizationArgs(group_size=-1, actorder=order)
        with pytest.raises(ValueError):
            QuantizationArgs(strategy="tensor", actorder=order)
    assert QuantizationArgs(group_size=1, actorder=True).actorder == A.GROUP
    assert QuantizationArgs(group_size=1, actorder=False).actorder is None
    assert QuantizationArgs(group_size=1, actorder=None).actorder is None
    assert QuantizationArgs(group_size=1, actorder="STATIC").actorder == A.WEIGHT
    with pytest.raises(ValueError):
        QuantizationArgs(group_size=1, actorder="sorted")


def test_patch_attr_restores_or_removes():
    obj = SimpleNamespace(a=1)
    with patch_attr(obj, "a", 2):
        assert obj.a == 2
    assert obj.a == 1
    with pytest.raises(RuntimeError):
        with patch_attr(obj, "b", 3):
            assert obj.b == 3
            raise RuntimeError()
    assert not hasattr(obj, "b")


def test_parameterized_default_dict():
    made = []

    def factory(size, kind="x", scale=1):
        made.append((size, kind, scale))
        return [size * scale, kind]

    d = ParameterizedDefaultDict(factory)
    assert d[3] == [3, "x"] and d[(4, "y")] == [4, "y"]
    first = d.get(5, factory_kwargs={"scale": 10})
    assert first == [50, "x"]
    # the keyword arguments are no part of the key: the entry made first stays
    assert d.get(5, factory_kwargs={"scale": 2}) is first
    assert d[(5,)] is first and made == [(3, "x", 1), (4, "y", 1), (5, "x", 10)]
    assert d._factory_kwargs == {}


def test_deprecated_warns_and_calls():
    @deprecated(future_name="new_name")
    def old_name(x):
        return x + 1

    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        assert old_name(1) == 2
    assert len(seen) == 1 and issubclass(seen[0].category, DeprecationWarning)
    assert "old_name is deprecated" in str(seen[0].message) and "new_name" in str(seen[0].message)

    @deprecated(message="gone soon")
    def other():
        return 0

    with pytest.warns(DeprecationWarning, match="gone soon"):
        other()


def test_module_helpers():
    assert fix_fsdp_module_name("a._fsdp_wrapped_module.b") == "a.b"
    assert fix_fsdp_module_name("a.b._fsdp_wrapped_module") == "a.b"
    assert fix_fsdp_module_name("_fsdp_wrapped_module.a") == "a"
    model = torch.nn.Sequential(torch.nn.Sequential(torch.nn.Linear(2, 2)), torch.nn.ReLU())
    new = torch.nn.Linear(2, 3)
    replace_module(model, "0.0", new)
    assert model[0][0] is new
    replace_module(model, "1", torch.nn.Tanh())
    assert isinstance(model[1], torch.nn.Tanh)
    assert is_compressed_tensors_config({"format": "dense"}) is False
    try:  # transformers builds one only where the reference's package is installed
        from transformers.utils.quantization_config import CompressedTensorsConfig

        config = CompressedTensorsConfig()
    except ImportError:
        return
    assert is_compressed_tensors_config(config) is True


def test_quantization_config_presets_and_calibration_needs():
    """quant_config.py:148-164, 262-278; tests/test_quantization/test_quant_config.py"""
    from compressed_tensors_amd.quantization import QuantizationConfig, QuantizationScheme

    config = QuantizationConfig(config_groups={"W4A16": ["Linear"], "w8a8": ["Conv2d"]})
    w4, w8 = config.config_groups["W4A16"], config.config_groups["w8a8"]
    assert isinstance(w4, QuantizationScheme) and w4.targets == ["Linear"] and w4.weights.num_bits == 4
    assert w4.input_activations is None and w8.targets == ["Conv2d"] and w8.input_activations.dynamic is True
    assert not config.requires_calibration_data()  # weights only, and inputs quantized per token on the fly
    assert config.to_dict() == config.model_dump()
    with pytest.raises(KeyError, match="Unknown preset scheme name"):
        QuantizationConfig(config_groups={"W5A5": ["Linear"]})

    static_in = QuantizationScheme(targets=["Linear"], weights=QuantizationArgs(),
                                   input_activations=QuantizationArgs(num_bits=8))
    assert QuantizationConfig(config_groups={"g": static_in}).requires_calibration_data()
    local = QuantizationScheme(targets=["Linear"], weights=QuantizationArgs(),
                               input_activations=QuantizationArgs(num_bits=4, type="float", strategy="tensor_group",
                                                                  group_size=16, dynamic="local"))
    assert QuantizationConfig(config_groups={"g": local}).requires_calibration_data()
    static_out = QuantizationScheme(targets=["Linear"], output_activations=QuantizationArgs(num_bits=8))
    assert QuantizationConfig(config_groups={"g": static_out}).requires_calibration_data()
    kv = QuantizationConfig(config_groups={"W4A16": ["Linear"]}, kv_cache_scheme={"num_bits": 8, "type": "float"})
    assert kv.requires_calibration_data() and kv.kv_cache_scheme.type == "float"
    assert QuantizationConfig.model_validate(kv.model_dump()) == kv
