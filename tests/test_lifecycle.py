"""Putting a quantization config on a model (host code; the kernels behind forward calls and
compress_quantized_weights are under the GPU tests): the behaviour of the reference's
quantization/lifecycle/apply.py:112-189, helpers.py:27-32 and utils/helpers.py:237-330, after its
tests/test_quantization/lifecycle/test_apply.py and test_enabled.py."""
import pytest
import torch

from compressed_tensors_amd.config import (BitmaskConfig, DenseSparsityConfig, QuantizationStatus,
                                           Sparse24BitMaskConfig)
from compressed_tensors_amd.linear.compressed_linear import CompressedLinear
from compressed_tensors_amd.quantization import (
    QuantizationArgs, QuantizationConfig, QuantizationScheme, apply_quantization_config,
    disable_quantization, enable_quantization, is_model_quantized, is_module_quantized,
    iter_named_leaf_modules, load_pretrained_quantization_parameters, module_type)
from compressed_tensors_amd.utils.safetensors_io import save_file


class Block(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.q_proj = torch.nn.Linear(32, 32, bias=False)
        self.up_proj = torch.nn.Linear(32, 64, bias=False)
        self.act = torch.nn.SiLU()


class Tiny(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.embed = torch.nn.Embedding(10, 32)
        self.layers = torch.nn.ModuleList([Block(), Block()])
        self.lm_head = torch.nn.Linear(32, 10, bias=False)


def _config(status="frozen", fmt="pack-quantized", inputs=None):
    scheme = QuantizationScheme(
        targets=["Linear"], weights=QuantizationArgs(num_bits=4, type="int", strategy="group", group_size=16),
        input_activations=inputs)
    other = QuantizationScheme(targets=["re:.*up_proj$"],
                               weights=QuantizationArgs(num_bits=8, type="int", strategy="channel", symmetric=False))
    return QuantizationConfig(config_groups={"group_0": other, "group_1": scheme}, format=fmt,
                              quantization_status=status, ignore=["lm_head"])


def test_apply_quantization_config():
    model = Tiny()
    assert not is_model_quantized(model)
    assert apply_quantization_config(model, None) == {}
    apply_quantization_config(model, _config())
    assert is_model_quantized(model)
    for block in model.layers:
        # up_proj matches both groups: the first target of the config decides
        assert block.up_proj.quantization_scheme.weights.num_bits == 8
        assert block.q_proj.quantization_scheme.weights.num_bits == 4
        assert block.q_proj.weight_scale.shape == (32, 2) and block.up_proj.weight_scale.shape == (64, 1)
        assert block.up_proj.weight_zero_point.dtype == torch.int8
        assert block.q_proj.quantization_status == QuantizationStatus.FROZEN
        assert hasattr(block.q_proj.forward.__func__, "_wraps_forward")
        assert not is_module_quantized(block.act)
    assert not is_module_quantized(model.lm_head) and not hasattr(model.lm_head, "weight_scale")
    assert not is_module_quantized(model.embed)
    assert module_type(model.lm_head) == "Linear"
    leaves = dict(iter_named_leaf_modules(model))
    assert "layers.0.q_proj" in leaves and "layers" not in leaves and "layers.0" not in leaves
    # a compressed status asks for no zero points on symmetric schemes
    model = Tiny()
    apply_quantization_config(model, _config(status="compressed"))
    assert not hasattr(model.layers[0].q_proj, "weight_zero_point")
    assert hasattr(model.layers[0].up_proj, "weight_zero_point")


def test_run_compressed_turns_linears_into_compressed_linears():
    model = Tiny()
    apply_quantization_config(model, _config(status="compressed"), run_compressed=True)
    q = model.layers[1].q_proj
    assert isinstance(q, CompressedLinear) and not hasattr(q, "weight")
    assert q.weight_packed.shape == (32, 4) and q.weight_packed.dtype == torch.int32
    assert q.quantization_status == QuantizationStatus.COMPRESSED
    assert type(model.lm_head) is torch.nn.Linear
    # the dense format leaves plain Linears
    model = Tiny()
    apply_quantization_config(model, _config(fmt="dense"), run_compressed=True)
    assert type(model.layers[0].q_proj) is torch.nn.Linear


def test_quantization_can_be_switched_off_per_module():
    """tests/test_quantization/lifecycle/test_enabled.py: a disabled module computes what the
    module did before it was wrapped"""
    model = Tiny()
    x = torch.randn(3, 32)
    want = model.layers[0].q_proj(x)
    apply_quantization_config(model, _config())
    model.apply(disable_quantization)
    assert model.layers[0].q_proj.quantization_enabled is False
    assert torch.equal(model.layers[0].q_proj(x), want)
    model.apply(enable_quantization)
    assert model.layers[0].q_proj.quantization_enabled is True
    # a second initialization does not wrap the wrapper
    first = model.layers[0].q_proj.forward.__func__._wraps_forward
    apply_quantization_config(model, _config())
    assert model.layers[0].q_proj.forward.__func__._wraps_forward is first


def test_load_pretrained_quantization_parameters(tmp_path):
    inputs = QuantizationArgs(num_bits=8, type="int", strategy="tensor", dynamic=False)
    model = Tiny()
    apply_quantization_config(model, _config(inputs=inputs))
    q = model.layers[0].q_proj
    stored = {
        "layers.0.q_proj.input_scale": torch.full_like(q.input_scale.data, 0.25),
        "layers.0.q_proj.weight_scale": torch.full_like(q.weight_scale.data, 0.5),
        "layers.0.q_proj.weight_zero_point": torch.ones_like(q.weight_zero_point.data),
        "layers.0.q_proj.weight": q.weight.data.clone(),
    }
    save_file(stored, str(tmp_path / "model.safetensors"))
    load_pretrained_quantization_parameters(model, str(tmp_path))
    assert torch.equal(q.input_scale.data, stored["layers.0.q_proj.input_scale"])
    assert torch.equal(q.input_zero_point.data, torch.zeros_like(q.input_zero_point.data))  # none stored: zeros
    assert not torch.equal(q.weight_scale.data, stored["layers.0.q_proj.weight_scale"])      # not asked for
    load_pretrained_quantization_parameters(model, str(tmp_path), load_weight_qparams=True)
    assert torch.equal(q.weight_scale.data, stored["layers.0.q_proj.weight_scale"])
    assert torch.equal(q.weight_zero_point.data, stored["layers.0.q_proj.weight_zero_point"])


def test_sparsity_config_classes():
    assert DenseSparsityConfig().format == "dense"
    assert BitmaskConfig(global_sparsity=0.7, targets=["Linear"]).format == "sparse-bitmask"
    s24 = Sparse24BitMaskConfig()
    assert s24.format == "sparse-24-bitmask" and s24.sparsity_structure == "2:4"


def test_statuses_compare_by_lifecycle_order_and_metadata_names():
    """quant_config.py:39-99, quant_metadata.py:24-62"""
    from compressed_tensors_amd.quantization import (DEFAULT_QUANTIZATION_FORMAT, DEFAULT_QUANTIZATION_METHOD,
                                                     LIFECYCLE_ORDER, KVCacheScaleType, QuantizationMetadata,
                                                     QuantizationScheme, QuantizationStatus,
                                                     is_kv_cache_quant_scheme)

    S = QuantizationStatus
    assert LIFECYCLE_ORDER == [S.INITIALIZED, S.CALIBRATION, S.FROZEN, S.COMPRESSED] == S.lifecycle_order()
    assert S.FROZEN > S.CALIBRATION and S.FROZEN >= S.FROZEN and S.INITIALIZED < S.COMPRESSED
    assert S.COMPRESSED <= S.COMPRESSED and not (S.CALIBRATION > S.FROZEN)
    # "compressed" sorts before "frozen" as a string: the order is the lifecycle's
    assert S.COMPRESSED > S.FROZEN
    assert S.INITIALIZED >= None and S.INITIALIZED > None and not (S.COMPRESSED < None) and not (S.COMPRESSED <= None)
    with pytest.raises(NotImplementedError):
        S.FROZEN > "calibration"
    assert S("frozen") is S.FROZEN and S.FROZEN == "frozen"
    assert (DEFAULT_QUANTIZATION_METHOD, DEFAULT_QUANTIZATION_FORMAT) == ("compressed-tensors", "fakequant")

    names = QuantizationMetadata.all_qparam_names()
    assert names[:2] == [KVCacheScaleType.KEY.value, KVCacheScaleType.VALUE.value] == ["k_scale", "v_scale"]
    assert len(names) == 14 and "weight_g_idx" in names and "input_global_scale" in names
    m = torch.nn.Linear(4, 4)
    m.weight_scale = torch.nn.Parameter(torch.ones(4, 1), requires_grad=False)
    m.k_scale = torch.nn.Parameter(torch.ones(1), requires_grad=False)
    m.other = torch.nn.Parameter(torch.ones(1), requires_grad=False)
    QuantizationMetadata.clear_all_qparams(m)
    assert sorted(n for n, _ in m.named_parameters()) == ["bias", "other", "weight"]

    assert is_kv_cache_quant_scheme(QuantizationScheme(targets=["re:.*self_attn$"]))
    assert not is_kv_cache_quant_scheme(QuantizationScheme(targets=["Linear"]))


def test_the_most_specific_target_decides_and_unmatched_targets_warn(caplog):
    """tests/test_quantization/lifecycle/test_apply.py:73-119, 312-344: a module's name beats a
    pattern, a pattern beats a class, whatever the order of the groups"""
    def group(bits, target):
        return {"weights": {"num_bits": bits}, "targets": [target]}

    config = QuantizationConfig(config_groups={
        "group_1": group(8, "Linear"), "group_2": group(4, "re:.*up_proj"),
        "group_3": group(2, "layers.0.up_proj"), "group_4": group(6, "re:.*foobarbaz")},
        ignore=["lm_head", "re:.*gate"])
    config.quantization_status = QuantizationStatus.CALIBRATION
    model = Tiny()
    with caplog.at_level("WARNING"):
        apply_quantization_config(model, config)
    # one target and one ignore entry name no module
    assert "Could not match `re:.*foobarbaz`" in caplog.text and caplog.text.count("Could not match") == 1
    bits = {name: m.quantization_scheme.weights.num_bits for name, m in model.named_modules()
            if hasattr(m, "quantization_scheme")}
    assert bits == {"layers.0.q_proj": 8, "layers.0.up_proj": 2, "layers.1.q_proj": 8, "layers.1.up_proj": 4}
    assert model.layers[0].q_proj.quantization_status == QuantizationStatus.CALIBRATION
    assert not hasattr(model.lm_head, "quantization_scheme")


def test_a_second_config_replaces_what_the_first_left():
    """tests/test_quantization/lifecycle/test_apply.py:347-442"""
    fp8 = QuantizationArgs(num_bits=8, type="float", strategy="tensor", symmetric=True, dynamic=False)
    first = QuantizationConfig(config_groups={"group_0": QuantizationScheme(
        targets=[r"re:.*(q|up)_proj$"], weights=fp8, input_activations=fp8)}, ignore=["lm_head"])
    second = QuantizationConfig(config_groups={"group_0": QuantizationScheme(
        targets=[r"re:.*up_proj$"],
        weights=QuantizationArgs(num_bits=4, type="int", strategy="group", group_size=16, symmetric=False))},
        ignore=["lm_head"])
    model = Tiny()
    apply_quantization_config(model, first)
    apply_quantization_config(model, second)
    for block in model.layers:
        up, q = block.up_proj, block.q_proj
        assert not hasattr(up, "input_scale") and not hasattr(up, "input_zero_point")
        assert up.weight_scale.shape == (64, 2) and up.weight_zero_point.shape == (64, 2)
        assert up.quantization_scheme.weights.num_bits == 4
        assert q.input_scale.shape == q.input_zero_point.shape == q.weight_scale.shape == (1,)
        assert q.quantization_scheme.weights.type == "float"
