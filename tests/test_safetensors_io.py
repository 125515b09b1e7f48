"""safetensors reader / writer and the config.json emitter: host logic, checked
against the safetensors library's own reader and writer (no GPU)."""
import json
import os

import pytest
import torch
from safetensors import safe_open
from safetensors.torch import load_file, save_file as official_save_file

from compressed_tensors_amd.utils.safetensors_io import (
    CheckpointReader,
    get_nested_weight_mappings,
    get_quantization_parameter_to_path_mapping,
    get_safetensors_header,
    get_weight_mappings,
    iter_tensors,
    save_file,
)


def _state():
    g = torch.Generator().manual_seed(3)
    return {
        "model.layers.0.q_proj.weight_packed": torch.randint(-2**31, 2**31 - 1, (16, 32), generator=g, dtype=torch.int64).to(torch.int32),
        "model.layers.0.q_proj.weight_scale": torch.randn(16, 2, generator=g).bfloat16(),
        "model.layers.0.q_proj.weight_shape": torch.tensor([16, 256]),
        "model.layers.0.q_proj.weight_zero_point": torch.randint(-8, 8, (2, 2), generator=g).to(torch.int32),
        "model.layers.0.k_proj.weight": torch.randn(4, 8, generator=g).to(torch.float8_e4m3fn),
        "model.layers.0.k_proj.weight_scale": torch.randn(4, 1, generator=g).half(),
        "model.norm.weight": torch.randn(7, generator=g),
        "lm_head.bitmask": torch.randint(0, 256, (3, 5), generator=g).to(torch.uint8),
        "flag": torch.tensor([True, False, True]),
        "scalar": torch.tensor(3.5, dtype=torch.float64),
        "empty": torch.empty(0, 4, dtype=torch.int8),
        "strided": torch.arange(24, dtype=torch.int16).reshape(4, 6).t(),
    }


def test_writer_matches_the_library(tmp_path):
    state = _state()
    mine, theirs = str(tmp_path / "mine.safetensors"), str(tmp_path / "theirs.safetensors")
    save_file(state, mine, metadata={"format": "pt"})
    official_save_file({k: v.contiguous() for k, v in state.items()}, theirs, metadata={"format": "pt"})
    loaded = load_file(mine)
    assert set(loaded) == set(state)
    for k, v in state.items():
        assert loaded[k].dtype == v.dtype and loaded[k].shape == v.shape, k
        assert torch.equal(loaded[k].reshape(-1).view(torch.uint8),
                           v.contiguous().reshape(-1).view(torch.uint8)), k
    # same header entries (dtype names, shapes, byte ranges) and same bytes as the library writes
    assert get_safetensors_header(mine) == get_safetensors_header(theirs)
    assert open(mine, "rb").read() == open(theirs, "rb").read()
    with safe_open(mine, framework="pt") as f:
        assert f.metadata() == {"format": "pt"}


def test_writer_streams_tensors_larger_than_its_staging_buffer(tmp_path):
    # host tensors do not go through the staging buffers, but the file layout code is shared
    state = {"a": torch.arange(100_000, dtype=torch.int32), "b": torch.arange(7, dtype=torch.uint8)}
    path = str(tmp_path / "x.safetensors")
    save_file(state, path, staging_bytes=4096)
    loaded = load_file(path)
    assert all(torch.equal(loaded[k], v) for k, v in state.items())
    with pytest.raises(ValueError):
        save_file({}, path)
    with pytest.raises(ValueError):
        save_file({"c": torch.zeros(2, dtype=torch.complex64)}, path)


def test_mappings_single_file_directory_and_index(tmp_path):
    state = _state()
    single = tmp_path / "single.safetensors"
    save_file(state, str(single))
    assert get_weight_mappings(str(single)) == {k: str(single) for k in state}

    d1 = tmp_path / "d1"
    d1.mkdir()
    save_file(state, str(d1 / "model.safetensors"))
    assert set(get_weight_mappings(str(d1)).values()) == {str(d1 / "model.safetensors")}

    d2 = tmp_path / "d2"
    d2.mkdir()
    names = sorted(state)
    shards = {"model-00001-of-00002.safetensors": names[::2], "model-00002-of-00002.safetensors": names[1::2]}
    weight_map = {}
    for fname, keys in shards.items():
        save_file({k: state[k] for k in keys}, str(d2 / fname))
        weight_map.update({k: fname for k in keys})
    (d2 / "model.safetensors.index.json").write_text(json.dumps({"metadata": {}, "weight_map": weight_map}))
    m = get_weight_mappings(str(d2))
    assert m == {k: str(d2 / v) for k, v in weight_map.items()}
    got = dict(iter_tensors(str(d2)))
    assert set(got) == set(state) and torch.equal(got["model.norm.weight"], state["model.norm.weight"])
    with CheckpointReader(str(d2)) as r:
        assert torch.equal(r.get("flag"), state["flag"])
        assert len(r._open) == 1
        r.get(names[0]), r.get(names[1])
        assert len(r._open) == 2
    with pytest.raises(KeyError):
        list(iter_tensors(str(d2), names=["nope"]))
    with pytest.raises(ValueError, match="Could not find"):
        get_weight_mappings(str(tmp_path))

    nested, rest = get_nested_weight_mappings(
        str(d2), ("weight_packed", "weight_scale", "weight_zero_point", "weight_shape"),
        return_unmatched_params=True)
    assert set(nested) == {"model.layers.0.q_proj", "model.layers.0.k_proj"}
    assert set(nested["model.layers.0.q_proj"]) == {"weight_packed", "weight_scale", "weight_zero_point", "weight_shape"}
    assert set(nested["model.layers.0.k_proj"]) == {"weight_scale"}
    assert "model.norm.weight" in rest and "model.layers.0.k_proj.weight" in rest
    q = get_quantization_parameter_to_path_mapping(str(d2))
    assert set(q) == {"model.layers.0.q_proj.weight_scale", "model.layers.0.q_proj.weight_zero_point",
                      "model.layers.0.k_proj.weight_scale"}


def test_update_config_and_back(tmp_path):
    from compressed_tensors_amd.compressors import ModelCompressor
    from compressed_tensors_amd.config import SparsityCompressionConfig
    from compressed_tensors_amd.quantization import QuantizationConfig, QuantizationScheme

    qc = QuantizationConfig(
        config_groups={"group_0": QuantizationScheme(
            targets=["Linear"], weights=dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128))},
        format="pack-quantized", ignore=["lm_head"])
    sc = SparsityCompressionConfig(format="sparse-24-bitmask", targets=["Linear"], sparsity_structure="2:4")
    (tmp_path / "config.json").write_text(json.dumps({"architectures": ["LlamaForCausalLM"], "hidden_size": 64}))
    mc = ModelCompressor(sparsity_config=sc, quantization_config=qc)
    mc.update_config(str(tmp_path))
    data = json.loads((tmp_path / "config.json").read_text())
    assert data["hidden_size"] == 64
    q = data["quantization_config"]
    assert q["quant_method"] == "compressed-tensors" and q["format"] == "pack-quantized"
    assert q["ignore"] == ["lm_head"] and "version" in q
    assert q["sparsity_config"]["format"] == "sparse-24-bitmask"
    w = q["config_groups"]["group_0"]["weights"]
    assert (w["num_bits"], w["strategy"], w["group_size"], w["symmetric"]) == (4, "group", 128, True)
    back = ModelCompressor.from_compression_config(q)
    assert back.quantization_config.model_dump() == qc.model_dump()
    assert back.sparsity_config.model_dump() == sc.model_dump()
    assert set(back.quantization_compressor) == {"pack-quantized"}
    assert ModelCompressor.from_compression_config(None) is None
    assert ModelCompressor.from_compression_config({"quant_method": "compressed-tensors"}) is None
    # nothing to write without any config
    os.remove(tmp_path / "config.json")
    ModelCompressor().update_config(str(tmp_path))
    assert not (tmp_path / "config.json").exists()


def test_helper_names_of_the_reference(tmp_path):
    """utils/safetensors_load.py: match_param_name :99-112, is_quantization_param :308-322,
    get_nested_mappings_from_state_dict :251-305, get_safetensors_folder :42-81 (local paths)"""
    from compressed_tensors_amd.utils.safetensors_io import (
        get_nested_mappings_from_state_dict, get_safetensors_folder, is_quantization_param, match_param_name)

    assert match_param_name("model.layers.0.q_proj.weight_scale", "weight_scale") == "model.layers.0.q_proj"
    assert match_param_name("model.layers.0.q_proj.weight_scale", "weight") is None
    assert match_param_name("weight_scale", "weight_scale") is None
    assert [is_quantization_param(n) for n in ("a.weight_scale", "a.input_zero_point", "a.weight_g_idx", "a.weight",
                                                "a.bitmask")] == [True, True, True, False, False]
    state = {"a.weight": torch.ones(1), "a.weight_scale": torch.ones(1), "b.bias": torch.ones(1)}
    nested, rest = get_nested_mappings_from_state_dict(state, ["weight", "weight_scale"], return_unmatched_params=True)
    assert set(nested) == {"a"} and set(nested["a"]) == {"weight", "weight_scale"} and set(rest) == {"b.bias"}
    assert get_nested_mappings_from_state_dict(state, ["bias"]) == {"b": {"bias": state["b.bias"]}}
    assert get_safetensors_folder(str(tmp_path)) == str(tmp_path.resolve())
