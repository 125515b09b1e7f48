"""Transform vocabulary and module matching on the host: what a config.json round trip keeps,
what the constructors refuse, and which modules a list of targets names (reference:
tests/test_transform/test_transform_args.py, test_transform_scheme.py,
test_transform_config.py, tests/test_utils/test_match.py)."""
import json

import pytest
import torch

from compressed_tensors_amd.transform import (TransformArgs, TransformConfig, TransformFactory,
                                              TransformLocation, TransformScheme)
from compressed_tensors_amd.utils import (InternalModule, is_match, is_narrow_match,
                                          match_modules_set, match_named_modules,
                                          match_named_parameters, match_targets)


def test_args_wrap_single_names_and_know_online_locations():
    a = TransformArgs(targets="Linear", location="input", ignore="lm_head")
    assert a.targets == ["Linear"] and a.ignore == ["lm_head"] and a.inverse is False
    assert a.location == TransformLocation.INPUT and a.is_online()
    assert not TransformArgs(targets=["x"], location="weight_output").is_online()
    assert TransformArgs(targets=["x"], location="k_cache").is_online()
    with pytest.raises(ValueError):
        TransformArgs(targets=["x"], location="weight")  # not a location of the enum
    with pytest.raises(ValueError):
        TransformArgs.model_validate({"targets": ["x"], "location": "input", "extra": 1})


def test_scheme_defaults_and_precision_names():
    s = TransformScheme(type="hadamard")
    assert s.apply == [] and not s.randomize and not s.requires_grad and s.head_dim is None
    assert s.precision is torch.float32
    assert TransformScheme(type="hadamard", precision="torch.float64").precision is torch.float64
    assert TransformScheme(type="hadamard", precision="bfloat16").precision is torch.bfloat16
    with pytest.raises(ValueError):
        TransformScheme(type="hadamard", precision="float63")
    with pytest.raises(ValueError):
        TransformScheme.model_validate({"type": "hadamard", "block_size": 16})
    # entries of `apply` may come as dictionaries
    s = TransformScheme(type="hadamard", apply=[{"targets": "Linear", "location": "input"}])
    assert isinstance(s.apply[0], TransformArgs) and s.apply[0].targets == ["Linear"]


def test_config_survives_json():
    config = TransformConfig(config_groups={
        "v": TransformScheme(type="random-hadamard", head_dim=128, precision=torch.float64,
                             apply=[TransformArgs(targets=["re:.*v_proj$"], location="weight_output"),
                                    TransformArgs(targets=["re:.*o_proj$"], location="weight_input",
                                                  inverse=True, ignore=["lm_head"])]),
        "r": TransformScheme(type="hadamard", randomize=True,
                             apply=[TransformArgs(targets="Linear", location="input")]),
    })
    text = json.dumps(config.model_dump())
    again = TransformConfig.model_validate(json.loads(text))
    assert again == config
    assert json.loads(text)["config_groups"]["v"]["precision"] == "torch.float64"
    assert json.loads(text)["config_groups"]["v"]["apply"][1] == {
        "targets": ["re:.*o_proj$"], "location": "weight_input", "inverse": True, "ignore": ["lm_head"]}
    with pytest.raises(ValueError):
        TransformConfig.model_validate({"config_groups": {}, "version": 2})


def test_factories_are_found_by_scheme_type():
    for kind, cls in (("hadamard", "HadamardFactory"), ("random-hadamard", "RandomHadamardFactory"),
                      ("random-matrix", "RandomMatrixFactory")):
        f = TransformFactory.from_scheme(TransformScheme(type=kind), name="t", seed=3)
        assert type(f).__name__ == cls and f.name == "t"
    with pytest.raises(Exception):
        TransformFactory.from_scheme(TransformScheme(type="fourier"), name="t")


# ------------------------------------------------------------------ matching
class Gate(torch.nn.Linear):
    pass


class Hooked(InternalModule):
    def __init__(self):
        super().__init__()
        self.inner = torch.nn.Linear(2, 2)


class Block(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.q_proj = torch.nn.Linear(4, 4)
        self.k_proj = torch.nn.Linear(4, 4)
        self.gate = Gate(4, 4)
        self.norm = torch.nn.LayerNorm(4)


class Tiny(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.layers = torch.nn.ModuleList([Block(), Block()])
        self.lm_head = torch.nn.Linear(4, 8)
        self.extra = Hooked()


def names(pairs):
    return [n for n, *_ in pairs]


def test_targets_are_names_patterns_or_classes_of_the_bases():
    m = Tiny()
    assert names(match_named_modules(m, ["layers.0.q_proj"])) == ["layers.0.q_proj"]
    assert names(match_named_modules(m, ["re:.*k_proj$"])) == ["layers.0.k_proj", "layers.1.k_proj"]
    # a subclass of Linear is a Linear; the module inside an InternalModule is an ordinary one,
    # the InternalModule itself never matches
    got = names(match_named_modules(m, ["Linear"], ignore=["lm_head", "re:.*k_proj"]))
    assert got == ["layers.0.q_proj", "layers.0.gate", "layers.1.q_proj", "layers.1.gate", "extra.inner"]
    assert names(match_named_modules(m, ["Gate"])) == ["layers.0.gate", "layers.1.gate"]
    assert names(match_named_modules(m, ["Hooked", "extra"])) == []
    assert names(match_named_modules(m, None)) == []
    # re.match anchors at the start only
    assert names(match_named_modules(m, ["re:layers.1"])) == [
        "layers.1", "layers.1.q_proj", "layers.1.k_proj", "layers.1.gate", "layers.1.norm"]
    assert is_match("lm_head", m.lm_head, "Linear") and not is_match("lm_head", m.lm_head, "Linear", "lm_head")
    assert not is_match("extra", m.extra, "re:.*")


def test_fused_names_stand_for_their_shards():
    m = torch.nn.ModuleDict({"qkv_proj": torch.nn.Identity()})
    fused = {"qkv_proj": ["q_proj", "k_proj", "v_proj"]}
    assert is_match("qkv_proj", m["qkv_proj"], "re:.*k_proj$", fused=fused)
    assert not is_match("qkv_proj", m["qkv_proj"], "re:.*k_proj$")
    assert not is_match("qkv_proj", m["qkv_proj"], "re:.*o_proj$", fused=fused)


def test_match_targets_orders_by_how_specific_a_target_is():
    m = Tiny()
    targets = ["Linear", "re:.*q_proj$", "layers.0.q_proj", "re:layers.*"]
    assert match_targets("layers.0.q_proj", m.layers[0].q_proj, targets) == [
        "layers.0.q_proj", "re:.*q_proj$", "re:layers.*", "Linear"]
    assert match_targets("extra", m.extra, ["re:.*"]) == []


def test_parameters_by_name_and_warning(caplog):
    m = Tiny()
    got = names(match_named_parameters(m, ["re:.*q_proj.weight$", "lm_head.bias"], ignore=["re:layers.1.*"]))
    assert got == ["layers.0.q_proj.weight", "lm_head.bias"]
    # one entry per target that names the parameter
    assert names(match_named_parameters(m, ["lm_head.bias", "re:lm_head.b.*"])) == ["lm_head.bias"] * 2
    with caplog.at_level("WARNING"):
        assert names(match_named_modules(m, ["nowhere"], warn_on_fail=True)) == []
    assert "Could not match `nowhere`" in caplog.text


def test_sets_of_modules_per_layer():
    m = Tiny()
    sets = list(match_modules_set(m, ["re:.*norm$", "re:.*q_proj$", "re:.*k_proj$"]))
    assert [[id(x) for x in s] for s in sets] == [
        [id(b.norm), id(b.q_proj), id(b.k_proj)] for b in m.layers]
    with pytest.raises(ValueError, match="twice"):
        list(match_modules_set(m, ["re:.*q_proj$", "lm_head"]))
    with pytest.raises(ValueError, match="Unable to match"):
        list(match_modules_set(m, ["lm_head", "re:.*no_such$"]))


def test_narrow_match():
    m = Tiny()
    assert is_narrow_match(m, "re:layers.0.*", "layers.0") is True
    assert is_narrow_match(m, "re:layers.0.*", "layers.0.q_proj") is False  # the parent matches too
    assert is_narrow_match(m, ["Linear"], "layers.0.q_proj") is True


@pytest.mark.parametrize("kind", ["hadamard", "random-hadamard"])
@pytest.mark.parametrize("randomize", [True, False])
def test_transforms_of_one_size_share_their_matrix(kind, randomize):
    """tests/test_transform/factory/test_memory.py:33-66: online transforms of the same size
    hold one matrix between them (here: none until a state dict asks, then one)"""
    from collections import Counter

    from compressed_tensors_amd.transform import TransformBase, apply_transform_config

    sizes = (2, 2, 4, 4, 8, 8)
    model = torch.nn.Sequential(*[torch.nn.Linear(a, b, bias=False) for a, b in zip(sizes, sizes[1:])])
    apply_transform_config(model, TransformConfig(config_groups={"": TransformScheme(
        type=kind, randomize=randomize, apply=[TransformArgs(targets="Linear", location="input"),
                                               TransformArgs(targets="Linear", location="output")])}))
    assert model.transform_config.config_groups[""].type == kind
    transforms = [m for m in model.modules() if isinstance(m, TransformBase)]
    assert len(transforms) == 10
    count = Counter(id(t.weight) for t in transforms)
    by_size = {t.weight.shape[0]: id(t.weight) for t in transforms}
    assert len(count) == len(by_size) == 3
    assert (count[by_size[2]], count[by_size[4]], count[by_size[8]]) == (3, 4, 3)
    state = model.state_dict()
    assert state["0._input.weight"].data_ptr() == state["1._input.weight"].data_ptr()
    assert ("0._input.perm" in state) == randomize
    for t in transforms:  # Hadamard: W W^T = n I
        w = t.weight.double()
        assert torch.equal(w @ w.T, w.shape[0] * torch.eye(w.shape[0], dtype=torch.float64))
