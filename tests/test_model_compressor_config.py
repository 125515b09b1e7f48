"""ModelCompressor's constructors and key lists (host code, no GPU): the cases of the reference's
tests/test_compressors/model_compressors/test_model_compressor.py:34-110 (config parsing),
:416-450 (several quantization formats in one model) and :453-505 (missing / unexpected keys),
with its literal configs."""
import json
from copy import deepcopy

import pytest
import torch

from compressed_tensors_amd.compressors import ModelCompressor
from compressed_tensors_amd.config import (CompressionFormat, SparsityCompressionConfig,
                                           infer_and_set_per_module_quantization_format)
from compressed_tensors_amd.quantization import QuantizationArgs, QuantizationConfig, QuantizationScheme


def sparsity_config():
    return {"format": "sparse-bitmask", "global_sparsity": 19.098103233975568,
            "registry_requires_subclass": False, "sparsity_structure": "unstructured"}


def quantization_config():
    return {
        "config_groups": {"group_0": {"targets": ["Linear"], "weights": {
            "num_bits": 4, "strategy": "channel", "symmetric": True, "type": "int"}}},
        "format": "pack-quantized", "global_compression_ratio": 1.891791164021256,
        "ignore": ["lm_head"], "quant_method": "compressed-tensors", "quantization_status": "frozen",
    }


def _combined(s_config, q_config):
    combined = deepcopy(q_config) if q_config is not None else {}
    if s_config is not None:
        combined["sparsity_config"] = s_config
    return combined


@pytest.mark.parametrize("s_config", [sparsity_config(), None])
@pytest.mark.parametrize("q_config", [quantization_config(), None])
def test_config_format(s_config, q_config):
    combined = _combined(s_config, q_config)
    assert ModelCompressor.parse_sparsity_config(combined) == s_config
    assert ModelCompressor.parse_quantization_config(combined) == q_config
    # metadata alone is no quantization config, an empty sparsity config is none
    assert ModelCompressor.parse_quantization_config(
        {"quant_method": "compressed-tensors", "version": "0.1", "sparsity_config": {}}) is None
    assert ModelCompressor.parse_sparsity_config({"sparsity_config": {}}) is None
    assert ModelCompressor.parse_sparsity_config(None) is None
    assert ModelCompressor.parse_quantization_config(None) is None


class _HFConfig:
    """stands in for transformers' CompressedTensorsConfig: the two configs as attributes"""

    def __init__(self, s_config, q_config):
        self.sparsity_config = (None if s_config is None
                                else SparsityCompressionConfig.load_from_registry(s_config["format"], **s_config))
        self.quantization_config = None if q_config is None else QuantizationConfig.model_validate(q_config)


@pytest.mark.parametrize("s_config,q_config", [(sparsity_config(), quantization_config()), (sparsity_config(), None),
                                               (None, quantization_config()), (None, None)])
@pytest.mark.parametrize("as_object", [False, True], ids=["dict", "object"])
def test_from_compression_config(s_config, q_config, as_object, tmp_path):
    combined = _combined(s_config, q_config)
    compressor = ModelCompressor.from_compression_config(_HFConfig(s_config, q_config) if as_object else combined)
    if s_config is None and q_config is None:
        assert compressor is None
        assert ModelCompressor.from_compression_config(None) is None
        return
    want_s = None if s_config is None else SparsityCompressionConfig.load_from_registry(s_config["format"], **s_config)
    want_q = None if q_config is None else QuantizationConfig.model_validate(q_config)
    assert compressor.sparsity_config == want_s
    assert compressor.quantization_config == want_q
    assert (compressor.sparsity_compressor is None) == (s_config is None)
    assert (compressor.quantization_compressor is None) == (q_config is None)
    if q_config is not None:
        assert list(compressor.quantization_compressor) == ["pack-quantized"]
    # the same through a config.json on disk, under either key, and back through update_config
    for key in ("quantization_config", "compression_config"):
        (tmp_path / "config.json").write_text(json.dumps({"model_type": "llama", key: combined}))
        for path in (tmp_path, tmp_path / "config.json"):
            loaded = ModelCompressor.from_pretrained(str(path))
            assert loaded.sparsity_config == want_s and loaded.quantization_config == want_q
    compressor.update_config(str(tmp_path))
    again = ModelCompressor.from_pretrained(str(tmp_path))
    assert again.sparsity_config == want_s and again.quantization_config == want_q
    assert json.loads((tmp_path / "config.json").read_text())["model_type"] == "llama"
    (tmp_path / "config.json").write_text(json.dumps({"model_type": "llama"}))
    assert ModelCompressor.from_pretrained(str(tmp_path)) is None


class TwoLayerModel(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.layer1 = torch.nn.Linear(10, 10, bias=False)
        self.layer2 = torch.nn.Linear(10, 10, bias=False)


def _int8_channel(fmt="int-quantized"):
    return QuantizationConfig.model_validate({
        "format": fmt, "global_compression_ratio": 1.0, "quant_method": "compressed-tensors",
        "config_groups": {"group_0": {"targets": ["Linear"], "weights": {
            "num_bits": 8, "strategy": "channel", "symmetric": True, "type": "int"}}}})


def _bitmask(targets):
    return SparsityCompressionConfig(format="sparse-bitmask", global_sparsity=0.7, targets=targets,
                                     sparsity_structure="unstructured")


def test_get_missing_keys():
    mc = ModelCompressor(sparsity_config=_bitmask(["re:.*layer1$"]), quantization_config=_int8_channel())
    assert sorted(mc.get_missing_module_keys(TwoLayerModel())) == ["layer1.weight"]
    # pack-quantized stores no `weight` for any quantized module either
    mc = ModelCompressor(sparsity_config=_bitmask(["re:.*layer1$"]),
                         quantization_config=_int8_channel("pack-quantized"))
    assert sorted(mc.get_missing_module_keys(TwoLayerModel())) == ["layer1.weight", "layer2.weight"]
    assert ModelCompressor(quantization_config=_int8_channel()).get_missing_module_keys(TwoLayerModel()) == []


def test_get_unexpected_keys():
    mc = ModelCompressor(sparsity_config=_bitmask(["re:.*layer1$"]), quantization_config=_int8_channel())
    expected = {f"{layer}.{suffix}" for layer, suffixes in {
        "layer1": ["shape", "row_offsets", "weight_zero_point", "weight_g_idx", "bitmask", "weight_scale",
                   "compressed"],
        "layer2": ["weight_scale", "weight_zero_point", "weight_g_idx"]}.items() for suffix in suffixes}
    actual = mc.get_unexpected_file_keys(TwoLayerModel())
    assert len(actual) == len(expected) and set(actual) == expected


def test_multiple_quant_compressors():
    model = torch.nn.Sequential(torch.nn.Linear(1, 2), torch.nn.Linear(2, 3))
    fp8 = QuantizationScheme(targets=["Linear"], weights=QuantizationArgs(num_bits=8, type="float"),
                             input_activations=QuantizationArgs(num_bits=8, type="float"),
                             format=CompressionFormat.float_quantized.value)
    nvfp4 = QuantizationScheme(targets=["Linear"], weights=QuantizationArgs(num_bits=4, type="float"),
                               input_activations=QuantizationArgs(num_bits=4, type="float"),
                               format=CompressionFormat.nvfp4_pack_quantized.value)
    model[0].quantization_scheme, model[0].quantization_status = fp8, "frozen"
    model[1].quantization_scheme, model[1].quantization_status = nvfp4, "frozen"
    compressor = ModelCompressor.from_pretrained_model(model, None)
    assert isinstance(compressor.quantization_compressor, dict)
    assert compressor.quantization_config.format == CompressionFormat.mixed_precision.value
    assert all(f in compressor.quantization_compressor for f in (fp8.format, nvfp4.format))
    assert list(compressor.quantization_config.config_groups) == ["group_0", "group_1"]


@pytest.mark.parametrize("weights,inputs,structure,want", [
    (dict(num_bits=4, type="int", strategy="group", group_size=128), None, None, "pack-quantized"),
    (dict(num_bits=8, type="int", strategy="channel"), None, None, "pack-quantized"),
    (dict(num_bits=4, type="int", strategy="group", group_size=128), None, "2:4", "marlin-24"),
    (dict(num_bits=4, type="int", strategy="tensor"), None, "2:4", "pack-quantized"),
    (dict(num_bits=8, type="float", strategy="channel"), None, None, "naive-quantized"),
    (dict(num_bits=8, type="float", strategy="channel"), dict(num_bits=8, type="float", dynamic=True, strategy="token"),
     None, "float-quantized"),
    (dict(num_bits=8, type="int", strategy="channel"), dict(num_bits=8, type="int", dynamic=True, strategy="token"),
     "2:4", "int-quantized"),
    (dict(num_bits=4, type="float", strategy="tensor_group", group_size=16), None, None, "nvfp4-pack-quantized"),
])
def test_inferred_formats(weights, inputs, structure, want):
    """config/format.py:32-84 case by case"""
    model = torch.nn.Sequential(torch.nn.Linear(4, 4), torch.nn.ReLU(), torch.nn.Linear(4, 4))
    for i in (0, 2):
        model[i].quantization_scheme = QuantizationScheme(
            targets=["Linear"], weights=QuantizationArgs(**weights),
            input_activations=None if inputs is None else QuantizationArgs(**inputs))
    assert infer_and_set_per_module_quantization_format(model, sparsity_structure=structure) == [want]
    assert model[0].quantization_scheme.format == want
    # a global format overrides; an unquantized model has none
    assert infer_and_set_per_module_quantization_format(model, quantization_format="naive-quantized") == ["naive-quantized"]
    assert infer_and_set_per_module_quantization_format(torch.nn.Sequential(torch.nn.Linear(2, 2))) is None


def test_quantization_config_from_a_model():
    """quantization/quant_config.py:166-260: groups, ignore list, status, format"""
    model = torch.nn.Sequential(torch.nn.Linear(4, 4), torch.nn.ReLU(), torch.nn.Linear(4, 4), torch.nn.Linear(4, 2))
    assert QuantizationConfig.from_pretrained(model) is None
    assert ModelCompressor.from_pretrained_model(model) is None
    scheme = QuantizationScheme(targets=["Linear"], weights=QuantizationArgs(num_bits=4, type="int", strategy="channel"))
    for i in (0, 2):
        model[i].quantization_scheme = QuantizationScheme(**{**scheme.model_dump()})
        model[i].quantization_status = "frozen"
    config = QuantizationConfig.from_pretrained(model)
    assert list(config.config_groups) == ["group_0"] and config.config_groups["group_0"] == scheme
    assert config.ignore == ["3"]          # a Linear without a scheme; ReLU and the container are no quantized type
    assert config.format == "dense" and config.quantization_status == "frozen"
    model[2].quantization_status = "compressed"
    assert QuantizationConfig.from_pretrained(model).format == "int-quantized"
    assert QuantizationConfig.from_pretrained(model, format=["pack-quantized"]).format == "pack-quantized"
    mc = ModelCompressor.from_pretrained_model(model, "sparse-24-bitmask", "pack-quantized")
    assert mc.sparsity_config.format == "sparse-24-bitmask"
    assert list(mc.quantization_compressor) == ["pack-quantized"] and mc.quantization_config.format == "pack-quantized"
