"""GPU: ModelCompressor on a small Llama-shaped module tree vs the oracle."""
import pytest
import torch

from gpu_util import announce, assert_bit_equal
from oracle import pack as op
from oracle import quant as oq
from oracle import sparse as osp

pytestmark = pytest.mark.gpu


class Block(torch.nn.Module):
    def __init__(self, d, f):
        super().__init__()
        self.q_proj = torch.nn.Linear(d, d, bias=False)
        self.k_proj = torch.nn.Linear(d, d // 4, bias=False)
        self.down_proj = torch.nn.Linear(f, d, bias=False)
        self.norm = torch.nn.LayerNorm(d)


class Tiny(torch.nn.Module):
    def __init__(self, d=256, f=512, layers=2):
        super().__init__()
        self.layers = torch.nn.ModuleList([Block(d, f) for _ in range(layers)])
        self.lm_head = torch.nn.Linear(d, 64, bias=False)


def _prepare(model, args, oargs, gpu):
    """calibrate with the GPU observer, keep a CPU copy for the oracle"""
    from compressed_tensors_amd.quantization import observe_weight_qparams

    cpu = {}
    for name, m in model.named_modules():
        if getattr(m, "quantization_scheme", None) is None:
            continue
        w = m.weight.data
        scale, zp = observe_weight_qparams(w, args)
        o_scale, o_zp = oq.observe_weight(w.cpu(), oargs)
        assert_bit_equal(scale, o_scale, "scale")
        m.register_parameter("weight_scale", torch.nn.Parameter(scale, requires_grad=False))
        m.register_parameter("weight_zero_point", torch.nn.Parameter(zp, requires_grad=False))
        cpu[name] = (w.cpu(), o_scale, o_zp)
    return cpu


@pytest.mark.parametrize("symmetric", [True, False])
def test_pack_quantized_model_roundtrip(symmetric, gpu):
    from compressed_tensors_amd.compressors import ModelCompressor, apply_quantization_scheme
    from compressed_tensors_amd.quantization import (
        QuantizationArgs, QuantizationConfig, QuantizationScheme,
    )

    announce("ModelCompressor pack-quantized", symmetric)
    torch.manual_seed(0)
    model = Tiny().to(torch.bfloat16).to(gpu)
    spec = dict(num_bits=4, type="int", symmetric=symmetric, strategy="group", group_size=128)
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    config = QuantizationConfig(
        config_groups={"g0": QuantizationScheme(targets=["Linear"], weights=args)},
        format="pack-quantized", ignore=["lm_head"])
    apply_quantization_scheme(model, config)
    cpu = _prepare(model, args, oargs, gpu)
    assert set(cpu) == {f"layers.{i}.{p}" for i in range(2) for p in ("q_proj", "k_proj", "down_proj")}

    mc = ModelCompressor(quantization_config=config)
    state = mc.compress(model)
    for name, (w, s, z) in cpu.items():
        want = op.pack_quantized_compress(w, s, oargs, zero_point=z)
        assert_bit_equal(state[f"{name}.weight_packed"], want["weight_packed"], name)
        assert state[f"{name}.weight_shape"].tolist() == list(w.shape)
        assert f"{name}.weight" not in state
        assert (f"{name}.weight_zero_point" in state) == (not symmetric)
    assert "lm_head.weight" in state and "layers.0.norm.weight" in state

    # in-memory: compress_model / decompress_model
    mc.compress_model(model)
    q = model.layers[0].q_proj
    assert hasattr(q, "weight_packed") and not hasattr(q, "weight")
    assert str(q.quantization_status.value) == "compressed"
    mc.decompress_model(model)
    for name, (w, s, z) in cpu.items():
        want = op.pack_quantized_compress(w, s, oargs, zero_point=z)
        data = dict(want, weight_scale=s)
        dense = op.pack_quantized_decompress(data, oargs)
        assert_bit_equal(model.get_submodule(name).weight.data, dense, f"{name} decompressed")

    # state-dict decompress into a fresh model
    fresh = Tiny().to(torch.bfloat16).to(gpu)
    apply_quantization_scheme(fresh, config)
    mc.decompress(state, fresh)
    for name, (w, s, z) in cpu.items():
        want = op.pack_quantized_compress(w, s, oargs, zero_point=z)
        dense = op.pack_quantized_decompress(dict(want, weight_scale=s), oargs)
        assert_bit_equal(fresh.get_submodule(name).weight.data, dense, f"{name} loaded")


def test_fp8_plus_sparse24_stack(gpu):
    """quantization first, sparsity second (float-quantized + sparse-24-bitmask)"""
    from compressed_tensors_amd.compressors import ModelCompressor, apply_quantization_scheme
    from compressed_tensors_amd.config import SparsityCompressionConfig
    from compressed_tensors_amd.quantization import (
        QuantizationArgs, QuantizationConfig, QuantizationScheme,
    )

    announce("ModelCompressor fp8 + 2:4")
    torch.manual_seed(1)
    model = Tiny(layers=1).to(torch.bfloat16).to(gpu)
    for m in model.modules():
        if isinstance(m, torch.nn.Linear):
            keep = osp.get_24_bytemasks(m.weight.data.cpu()).to(gpu)
            m.weight.data = torch.where(keep, m.weight.data, torch.zeros_like(m.weight.data))
    spec = dict(num_bits=8, type="float", symmetric=True, strategy="channel")
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    qcfg = QuantizationConfig(
        config_groups={"g0": QuantizationScheme(targets=["Linear"], weights=args)},
        format="float-quantized", ignore=["lm_head"])
    scfg = SparsityCompressionConfig(format="sparse-24-bitmask", targets=["Linear"],
                                     ignore=["lm_head"], sparsity_structure="2:4")
    apply_quantization_scheme(model, qcfg)
    cpu = _prepare(model, args, oargs, gpu)
    mc = ModelCompressor(sparsity_config=scfg, quantization_config=qcfg)
    # every targeted Linear goes through the kernel that quantizes and compresses in one pass
    assert set(mc._compress_quantized_24(model, model.state_dict())) == {f"{n}.weight" for n in cpu}
    state = mc.compress(model)
    for name, (w, s, z) in cpu.items():
        codes = op.naive_compress(w, s, oargs, zero_point=z)
        vals, bm = osp.sparse24_bitmask_compress(codes)
        assert_bit_equal(state[f"{name}.compressed"], vals, f"{name}.compressed")
        assert_bit_equal(state[f"{name}.bitmask"], bm, f"{name}.bitmask")
        assert state[f"{name}.shape"].flatten().tolist() == list(w.shape)
        assert f"{name}.weight" not in state and f"{name}.weight_scale" in state
    # the way back, from the state dict: every such module through the kernel that decompresses
    # and dequantizes in one pass
    import copy
    from unittest import mock

    want = {}
    for name, (w, s, z) in cpu.items():
        codes = op.naive_compress(w, s, oargs, zero_point=z)
        want[name] = op.naive_decompress({"weight": codes, "weight_scale": s})
    other = copy.deepcopy(model)
    for name in cpu:
        other.get_submodule(name).weight.data.zero_()
    from compressed_tensors_amd.compressors import sparse_24_bitmask as s24

    taken = []

    def spy(recs, inner=s24.sparse24_decompress_dequantize_many):
        out = inner(recs)
        taken.extend(o is not None for o in out)
        return out

    with mock.patch.object(s24, "sparse24_decompress_dequantize_many", spy):
        mc.decompress(dict(state), other)
    assert len(taken) == len(cpu) and all(taken)  # every module through the one-pass kernel
    for name in cpu:
        assert_bit_equal(other.get_submodule(name).weight.data, want[name], f"{name} from the state dict")
        assert_bit_equal(other.get_submodule(name).weight_scale.data, cpu[name][1], f"{name}.weight_scale")
    # ... and in memory
    mc.compress_model(model)
    for name, (w, s, z) in cpu.items():
        module = model.get_submodule(name)
        assert_bit_equal(module.compressed.data, state[f"{name}.compressed"], f"{name}.compressed in memory")
        assert_bit_equal(module.bitmask.data, state[f"{name}.bitmask"], f"{name}.bitmask in memory")
        assert not hasattr(module, "weight")
    taken.clear()
    with mock.patch.object(s24, "sparse24_decompress_dequantize_many", spy):
        mc.decompress_model(model)
    assert len(taken) == len(cpu) and all(taken)  # every module through the one-pass kernel
    for name in cpu:
        assert_bit_equal(model.get_submodule(name).weight.data, want[name], f"{name} decompressed")


@pytest.mark.parametrize("fmt,spec,dtype", [
    ("pack-quantized", dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128), torch.bfloat16),
    ("pack-quantized", dict(num_bits=4, type="int", symmetric=False, strategy="channel"), torch.float16),
    ("float-quantized", dict(num_bits=8, type="float", symmetric=True, strategy="channel"), torch.bfloat16),
    ("nvfp4-pack-quantized", dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16), torch.bfloat16),
], ids=["w4a16", "w4a16-asym-channel", "fp8", "nvfp4"])
def test_compressed_linear_runs_from_compressed_parameters(fmt, spec, dtype, gpu):
    """CompressedLinear.from_linear gives empty parameters of the compressed shapes;
    filled from a compressed state dict, the first forward decompresses (on the GPU)
    and every forward equals a Linear holding the oracle's decompressed weight"""
    from compressed_tensors_amd import CompressedLinear
    from compressed_tensors_amd.compressors import BaseCompressor
    from compressed_tensors_amd.config import QuantizationStatus
    from compressed_tensors_amd.quantization import QuantizationArgs, QuantizationScheme

    announce("CompressedLinear", fmt, spec, dtype)
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    g = torch.Generator().manual_seed(12)
    w = (torch.randn(96, 256, generator=g) * 0.02).to(dtype)
    bias = torch.randn(96, generator=g).to(dtype)
    gs = None
    if spec["strategy"] == "tensor_group":
        gs = oq.generate_gparam(*[t.reshape(1) for t in torch.aminmax(w)])
    scale, zp = oq.observe_weight(w, oargs, global_scale=gs)
    if fmt == "pack-quantized":
        compressed = op.pack_quantized_compress(w, scale, oargs, zero_point=zp)
        compressed["weight_scale"] = scale
        dense = op.pack_quantized_decompress(dict(compressed), oargs)
    elif fmt == "float-quantized":
        compressed = dict(weight=op.naive_compress(w, scale, oargs, zero_point=zp), weight_scale=scale)
        dense = op.naive_decompress(dict(compressed))
    else:
        compressed = {"weight_packed": op.nvfp4_compress(w, scale, gs, oargs), "weight_scale": scale,
                      "weight_global_scale": gs}
        dense = op.nvfp4_decompress(compressed["weight_packed"], scale, gs)

    layer = torch.nn.Linear(256, 96, bias=True).to(dtype).to(gpu)
    layer.bias.data.copy_(bias)
    scheme = QuantizationScheme(targets=["Linear"], weights=args)
    with pytest.warns(UserWarning):
        CompressedLinear(4, 4)
    module = CompressedLinear.from_linear(layer, scheme, fmt)
    assert isinstance(module, CompressedLinear) and module is layer
    assert module.quantization_status == QuantizationStatus.COMPRESSED
    info = BaseCompressor.load_from_registry(fmt).compression_param_info(w.shape, args)
    assert ("weight" in info) == hasattr(module, "weight")  # the naive formats keep the name
    for name, (shape, pdtype) in info.items():
        p = getattr(module, name)
        assert tuple(p.shape) == tuple(shape) and p.dtype == pdtype and p.device.type == "cuda"
    assert module.weight_scale.shape == scale.shape and module.weight_scale.dtype == scale.dtype
    for name, value in compressed.items():  # what loading a checkpoint does
        assert tuple(getattr(module, name).shape) == tuple(value.shape), name
        getattr(module, name).data.copy_(value.to(gpu))

    x = torch.randn(5, 256, generator=g).to(dtype).to(gpu)
    want = torch.nn.functional.linear(x, dense.to(dtype).to(gpu), bias.to(gpu))
    for _ in range(2):
        got = module(x)
        assert module.quantization_status == QuantizationStatus.FROZEN
        assert_bit_equal(got, want.cpu(), "forward")
    assert_bit_equal(module.weight.data, dense.to(module.weight.dtype), "decompressed weight")


def test_checkpoint_on_disk_roundtrip(tmp_path, gpu):
    """compress on the GPU -> stream into a safetensors file (tensors bigger than the
    staging buffers) + config.json -> a fresh process-side view: the library's own reader
    sees the same tensors, and decompress(path, model) restores the oracle's weights"""
    import json

    from safetensors.torch import load_file

    from compressed_tensors_amd.compressors import (
        ModelCompressor, apply_quantization_scheme, load_compressed, save_compressed,
    )
    from compressed_tensors_amd.config import SparsityCompressionConfig
    from compressed_tensors_amd.quantization import (
        QuantizationArgs, QuantizationConfig, QuantizationScheme,
    )
    from compressed_tensors_amd.utils.safetensors_io import save_file

    announce("checkpoint on disk")
    torch.manual_seed(4)
    model = Tiny().to(torch.bfloat16).to(gpu)
    spec = dict(num_bits=4, type="int", symmetric=False, strategy="group", group_size=128)
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    config = QuantizationConfig(
        config_groups={"g0": QuantizationScheme(targets=["Linear"], weights=args)},
        format="pack-quantized", ignore=["lm_head"])
    apply_quantization_scheme(model, config)
    cpu = _prepare(model, args, oargs, gpu)
    mc = ModelCompressor(quantization_config=config)
    state = mc.compress(model)
    assert all(t.is_cuda for t in state.values() if t.numel() > 2)

    path = tmp_path / "model.safetensors"
    save_file(state, str(path), metadata={"format": "pt"}, staging_bytes=4096)  # many pieces per tensor
    mc.update_config(str(tmp_path))
    on_disk = load_file(str(path))
    assert set(on_disk) == set(state)
    for k, v in state.items():
        assert_bit_equal(on_disk[k], v.cpu(), k)

    q = json.loads((tmp_path / "config.json").read_text())["quantization_config"]
    loaded_mc = ModelCompressor.from_compression_config(q)
    fresh = Tiny().to(torch.bfloat16).to(gpu)
    apply_quantization_scheme(fresh, loaded_mc.quantization_config)
    loaded_mc.decompress(str(tmp_path), fresh)
    for name, (w, s, z) in cpu.items():
        want = op.pack_quantized_compress(w, s, oargs, zero_point=z)
        dense = op.pack_quantized_decompress(dict(want, weight_scale=s), oargs)
        assert_bit_equal(fresh.get_submodule(name).weight.data, dense, f"{name} from disk")

    # the sparse helpers: save_compressed / load_compressed through a file
    w = torch.randn(64, 96, device=gpu).bfloat16()
    w = torch.where(torch.rand_like(w.float()) < 0.6, torch.zeros_like(w), w)
    sparse_path = tmp_path / "sparse.safetensors"
    save_compressed({"a.weight": w, "b.bias": torch.ones(3, device=gpu)}, sparse_path, "sparse-bitmask")
    assert set(load_file(str(sparse_path))) == {"a.compressed", "a.bitmask", "a.shape", "a.row_offsets", "b.bias"}
    back = dict(load_compressed(sparse_path, SparsityCompressionConfig(format="sparse-bitmask"),
                                device=str(gpu)))
    assert_bit_equal(back["a.weight"], w.cpu(), "sparse round trip through a file")
    assert_bit_equal(back["b.bias"], torch.ones(3), "passed through")
    dense_back = dict(load_compressed(sparse_path, None))
    assert set(dense_back) == {"a.compressed", "a.bitmask", "a.shape", "a.row_offsets", "b.bias"}
    with pytest.raises(ValueError):
        save_compressed({}, sparse_path, "sparse-bitmask")
    with pytest.raises(ValueError, match="Unknown compression format"):
        save_compressed({"a.weight": w}, sparse_path, "no-such-format")


def test_forward_runs_after_compress_and_decompress_model(gpu):
    """Linear(bias=False) keeps its empty `bias` slot through compress_model and
    decompress_model: forward reads it.  The decompressed model computes with the
    oracle's weights."""
    from compressed_tensors_amd.compressors import ModelCompressor, apply_quantization_scheme
    from compressed_tensors_amd.quantization import (
        QuantizationArgs, QuantizationConfig, QuantizationScheme,
    )

    announce("forward after compress_model + decompress_model")
    torch.manual_seed(2)
    model = Tiny().to(torch.bfloat16).to(gpu)
    spec = dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128)
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    config = QuantizationConfig(
        config_groups={"g0": QuantizationScheme(targets=["Linear"], weights=args)},
        format="pack-quantized", ignore=["lm_head"])
    apply_quantization_scheme(model, config)
    cpu = _prepare(model, args, oargs, gpu)
    mc = ModelCompressor(quantization_config=config)
    for _ in range(2):  # the second round starts from modules that still hold the packed words
        mc.compress_model(model)
        for name in cpu:
            m = model.get_submodule(name)
            assert "bias" in m._parameters and m.bias is None
            assert set(n for n, p in m._parameters.items() if p is not None) == {
                "weight_packed", "weight_shape", "weight_scale"}
        mc.decompress_model(model)
    x = torch.randn(3, 256, device=gpu).bfloat16()
    for name, (w, s, z) in cpu.items():
        m = model.get_submodule(name)
        assert "bias" in m._parameters and m.bias is None
        want = op.pack_quantized_compress(w, s, oargs, zero_point=z)
        dense = op.pack_quantized_decompress(dict(want, weight_scale=s), oargs)
        assert_bit_equal(m.weight.data, dense, name)
        xin = x if m.in_features == 256 else torch.randn(3, m.in_features, device=gpu).bfloat16()
        assert_bit_equal(m(xin), torch.nn.functional.linear(xin, dense.to(gpu)).cpu(), f"{name} forward")


def test_module_pathway_equals_state_dict_pathway(gpu):
    """compress_model (job tables written by columns for the common case) leaves in every
    module what compress(state_dict) returns for it - for the weights that take the common
    path and for those that do not (asymmetric, activation ordering, channel strategy, fp32)"""
    from compressed_tensors_amd.compressors import ModelCompressor, apply_quantization_scheme
    from compressed_tensors_amd.quantization import (
        QuantizationArgs, QuantizationConfig, QuantizationScheme, observe_weight_qparams,
    )

    announce("compress_model vs compress(state_dict)")
    torch.manual_seed(3)

    class Mixed(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.a = torch.nn.ModuleList([torch.nn.Linear(256, 64 + 8 * i, bias=False) for i in range(11)])
            self.b = torch.nn.ModuleList([torch.nn.Linear(256, 48, bias=True) for _ in range(3)])   # asymmetric
            self.c = torch.nn.ModuleList([torch.nn.Linear(384, 40, bias=False) for _ in range(2)])  # channel
            self.d = torch.nn.Linear(256, 24, bias=False)                                           # g_idx
            self.e = torch.nn.Linear(128, 16, bias=False)                                           # fp32 weight

    model = Mixed().to(torch.bfloat16).to(gpu)
    model.e.float()
    sym = QuantizationArgs(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128)
    asym = QuantizationArgs(num_bits=4, type="int", symmetric=False, strategy="group", group_size=64)
    chan = QuantizationArgs(num_bits=8, type="int", symmetric=True, strategy="channel")
    config = QuantizationConfig(config_groups={
        "sym": QuantizationScheme(targets=["re:a\\..*", "d", "e"], weights=sym),
        "asym": QuantizationScheme(targets=["re:b\\..*"], weights=asym),
        "chan": QuantizationScheme(targets=["re:c\\..*"], weights=chan)}, format="pack-quantized")
    apply_quantization_scheme(model, config)
    for name, m in model.named_modules():
        scheme = getattr(m, "quantization_scheme", None)
        if scheme is None:
            continue
        w = m.weight.data
        g_idx = None
        if name == "d":
            g_idx = (torch.randperm(256, device=gpu) // 128).to(torch.int32)
            w = w.index_select(1, torch.argsort(g_idx.long()))
            m.register_parameter("weight_g_idx", torch.nn.Parameter(g_idx, requires_grad=False))
        scale, zp = observe_weight_qparams(w, scheme.weights)
        m.register_parameter("weight_scale", torch.nn.Parameter(scale, requires_grad=False))
        m.register_parameter("weight_zero_point", torch.nn.Parameter(zp, requires_grad=False))
    mc = ModelCompressor(quantization_config=config)
    want = mc.compress(model)
    dense_before = {n: p.data.clone() for n, p in model.named_parameters() if n.endswith(".weight")}
    mc.compress_model(model)
    got = {n: p.data for n, p in model.named_parameters()}
    assert set(got) == set(want)
    for name in want:
        assert_bit_equal(got[name], want[name].to(got[name].device), name)
    assert model.b[0].bias is not None and model.a[0].bias is None and "bias" in model.a[0]._parameters
    # ... and back: every weight equals its per-weight decompression
    packed = {n: p.data for n, p in model.named_parameters()}
    mc.decompress_model(model)
    comp = mc.quantization_compressor["pack-quantized"]
    for name, m in model.named_modules():
        scheme = getattr(m, "quantization_scheme", None)
        if scheme is None:
            continue
        data = {k[len(name) + 1:]: v for k, v in packed.items() if k.startswith(name + ".")}
        single = comp.decompress_weight(compressed_data=data, quantization_args=scheme.weights)
        assert_bit_equal(m.weight.data, single.cpu(), f"{name} decompressed")
        assert m.weight.dtype == m.weight_scale.dtype
        assert dense_before[f"{name}.weight"].shape == m.weight.shape


@pytest.mark.parametrize("fmt,spec", [
    ("float-quantized", dict(num_bits=8, type="float", symmetric=True, strategy="channel")),
    ("int-quantized", dict(num_bits=8, type="int", symmetric=False, strategy="group", group_size=64)),
    ("int-quantized", dict(num_bits=8, type="int", symmetric=True, strategy="tensor")),
    ("nvfp4-pack-quantized", dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16)),
], ids=["fp8-channel", "int8-asym-group", "int8-tensor", "nvfp4"])
def test_module_pathway_of_the_other_formats(fmt, spec, gpu):
    """compress_model / decompress_model for the int8 / fp8 and nvfp4 formats (job tables written
    by columns): the same parameters as compress(state_dict) leaves, codes equal to the oracle's,
    dense weights equal to the per-weight decompression; modules the table does not take
    (activation ordering, a bias-carrying one, an fp32 one) among them; forward runs afterwards"""
    from compressed_tensors_amd.compressors import ModelCompressor, apply_quantization_scheme
    from compressed_tensors_amd.quantization import (
        QuantizationArgs, QuantizationConfig, QuantizationScheme, observe_weight_qparams,
    )
    from compressed_tensors_amd.quantization.helpers import generate_gparam

    announce("module pathway", fmt, spec)
    torch.manual_seed(7)

    class Mixed(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.a = torch.nn.ModuleList([torch.nn.Linear(256, 64 + 16 * i, bias=False) for i in range(9)])
            self.b = torch.nn.ModuleList([torch.nn.Linear(128, 48, bias=True) for _ in range(3)])
            self.c = torch.nn.Linear(256, 32, bias=False)   # activation ordering (where the format has it)
            self.e = torch.nn.Linear(128, 16, bias=False)   # fp32 weight

    model = Mixed().to(torch.bfloat16).to(gpu)
    model.e.float()
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    config = QuantizationConfig(
        config_groups={"g0": QuantizationScheme(targets=["Linear"], weights=args)}, format=fmt)
    apply_quantization_scheme(model, config)
    nvfp4 = spec["strategy"] == "tensor_group"
    grouped = spec["strategy"] == "group"
    oracle_in = {}
    for name, m in model.named_modules():
        if getattr(m, "quantization_scheme", None) is None:
            continue
        w = m.weight.data
        gs = None
        if nvfp4:
            mn, mx = torch.aminmax(w)
            gs = generate_gparam(mn.reshape(1), mx.reshape(1))
            m.register_parameter("weight_global_scale", torch.nn.Parameter(gs, requires_grad=False))
        scale, zp = observe_weight_qparams(w, args, global_scale=gs) if nvfp4 else observe_weight_qparams(w, args)
        m.register_parameter("weight_scale", torch.nn.Parameter(scale, requires_grad=False))
        m.register_parameter("weight_zero_point", torch.nn.Parameter(zp, requires_grad=False))
        if name == "c" and grouped:
            g_idx = (torch.randperm(256, device=gpu) // 64).to(torch.int32)
            m.register_parameter("weight_g_idx", torch.nn.Parameter(g_idx, requires_grad=False))
        elif name != "c":
            oracle_in[name] = (w.cpu(), scale.cpu(), zp.cpu(), None if gs is None else gs.cpu())
    mc = ModelCompressor(quantization_config=config)
    want = mc.compress(model)
    # (compress(model) enqueues from the modules before it builds the state dict; given the
    # state dict it cannot: same entries, same order)
    given = mc.compress(model, state_dict=model.state_dict())
    assert list(given) == list(want)
    for name in want:
        assert_bit_equal(given[name], want[name].to(given[name].device), f"{name} from a given state dict")
    mc.compress_model(model)
    got = {n: p.data for n, p in model.named_parameters()}
    assert set(got) == set(want)
    for name in want:
        assert_bit_equal(got[name], want[name].to(got[name].device), name)
    assert model.b[0].bias is not None and model.a[0].bias is None and "bias" in model.a[0]._parameters
    for name, (w, s, z, gs) in oracle_in.items():
        if nvfp4:
            assert_bit_equal(got[f"{name}.weight_packed"], op.nvfp4_compress(w, s, gs, oargs), f"{name} codes")
        else:
            assert_bit_equal(got[f"{name}.weight"], op.naive_compress(w, s, oargs, zero_point=z), f"{name} codes")
    compressed = {n: p.data for n, p in model.named_parameters()}
    mc.decompress_model(model)
    comp = mc.quantization_compressor[fmt]
    for name, m in model.named_modules():
        scheme = getattr(m, "quantization_scheme", None)
        if scheme is None:
            continue
        data = {k[len(name) + 1:]: v for k, v in compressed.items() if k.startswith(name + ".")}
        single = comp.decompress_weight(compressed_data=data, quantization_args=scheme.weights)
        assert_bit_equal(m.weight.data, single.cpu(), f"{name} decompressed")
        assert m.weight.dtype == single.dtype and m.weight.shape == single.shape
        x = torch.randn(2, m.in_features, device=gpu).to(m.weight.dtype)
        assert_bit_equal(m(x), torch.nn.functional.linear(x, single, m.bias).cpu(), f"{name} forward")
    # a second round starts from modules that hold both the codes' leftovers and the dense weight
    mc.compress_model(model)
    again = {n: p.data for n, p in model.named_parameters()}
    assert set(again) == set(want)


@pytest.mark.parametrize("fmt", ["sparse-24-bitmask", "sparse-bitmask"])
def test_sparsity_only_model_in_memory(fmt, gpu):
    """compress_model / decompress_model with a sparsity compressor alone (the targets of a
    batch share one call of the compressor): the modules hold what compress(model) returns,
    the way back is lossless, forward runs"""
    from compressed_tensors_amd.compressors import ModelCompressor
    from compressed_tensors_amd.config import SparsityCompressionConfig

    announce("sparsity-only model", fmt)
    torch.manual_seed(9)
    model = Tiny(layers=2).to(torch.bfloat16).to(gpu)
    dense = {}
    for name, m in model.named_modules():
        if isinstance(m, torch.nn.Linear):
            keep = osp.get_24_bytemasks(m.weight.data.cpu()).to(gpu)
            m.weight.data = torch.where(keep, m.weight.data, torch.zeros_like(m.weight.data))
            dense[name] = m.weight.data.clone()
    scfg = SparsityCompressionConfig(format=fmt, targets=["Linear"], ignore=["lm_head"],
                                     sparsity_structure="2:4" if fmt == "sparse-24-bitmask" else "unstructured")
    mc = ModelCompressor(sparsity_config=scfg)
    want = mc.compress(model)
    mc.compress_model(model)
    got = {n: p.data for n, p in model.named_parameters()}
    assert set(got) == set(want)
    for name in want:
        assert_bit_equal(got[name], want[name].to(got[name].device), name)
    for name in dense:
        if name == "lm_head":
            continue
        values, bitmask = (osp.sparse24_bitmask_compress(dense[name].cpu()) if fmt == "sparse-24-bitmask"
                           else osp.bitmask_compress(dense[name].cpu())[:2])
        assert_bit_equal(got[f"{name}.compressed"], values, f"{name}.compressed")
        assert_bit_equal(got[f"{name}.bitmask"], bitmask, f"{name}.bitmask")
        assert not hasattr(model.get_submodule(name), "weight")
    mc.decompress_model(model)
    for name, w in dense.items():
        m = model.get_submodule(name)
        assert_bit_equal(m.weight.data, w.cpu(), f"{name} restored")
        x = torch.randn(2, m.in_features, device=gpu).bfloat16()
        assert_bit_equal(m(x), torch.nn.functional.linear(x, w).cpu(), f"{name} forward")


@pytest.mark.parametrize("fmt", ["pack-quantized", "int-quantized", "float-quantized", "nvfp4-pack-quantized"])
def test_module_pathway_on_a_seeded_mixture(fmt, gpu):
    """40 Linear modules of mixed shapes (some whose outputs cannot share an allocation), dtypes
    and schemes in one model: compress_model leaves in every module what compress_weight gives
    for it alone, decompress_model what decompress_weight gives"""
    import random

    from compressed_tensors_amd.compressors import ModelCompressor, apply_quantization_scheme
    from compressed_tensors_amd.quantization import (
        QuantizationArgs, QuantizationConfig, QuantizationScheme, observe_weight_qparams,
    )
    from compressed_tensors_amd.quantization.helpers import generate_gparam

    announce("seeded mixture", fmt)
    rng = random.Random(fmt)
    torch.manual_seed(len(fmt))
    if fmt == "pack-quantized":
        specs = [dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128),
                 dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=32),
                 dict(num_bits=8, type="int", symmetric=True, strategy="channel"),
                 dict(num_bits=4, type="int", symmetric=False, strategy="group", group_size=64)]
    elif fmt == "int-quantized":
        specs = [dict(num_bits=8, type="int", symmetric=True, strategy="channel"),
                 dict(num_bits=8, type="int", symmetric=False, strategy="group", group_size=32),
                 dict(num_bits=8, type="int", symmetric=True, strategy="tensor")]
    elif fmt == "float-quantized":
        specs = [dict(num_bits=8, type="float", symmetric=True, strategy="channel"),
                 dict(num_bits=8, type="float", symmetric=True, strategy="group", group_size=128),
                 dict(num_bits=8, type="float", symmetric=True, strategy="block", block_structure=[16, 64])]
    else:
        specs = [dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16)]
    ins, outs = [128, 256, 384, 1024], [16, 24, 40, 64, 72, 200]
    model = torch.nn.Module()
    model.m = torch.nn.ModuleList()
    groups = {}
    for i in range(40):
        spec = specs[rng.randrange(len(specs))]
        dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
        if fmt == "nvfp4-pack-quantized":
            dtype = rng.choice([torch.bfloat16, torch.float16])
        lin = torch.nn.Linear(rng.choice(ins), rng.choice(outs), bias=rng.random() < 0.3).to(dtype).to(gpu)
        if spec.get("strategy") == "block":
            lin = torch.nn.Linear(rng.choice([128, 256]), rng.choice([16, 64]), bias=False).to(dtype).to(gpu)
        model.m.append(lin)
        groups.setdefault(tuple(sorted((k, str(v)) for k, v in spec.items())), (spec, []))[1].append(f"m.{i}")
    config = QuantizationConfig(config_groups={
        f"g{k}": QuantizationScheme(targets=names, weights=QuantizationArgs(**spec))
        for k, (spec, names) in enumerate(groups.values())}, format=fmt)
    apply_quantization_scheme(model, config)
    mc = ModelCompressor(quantization_config=config)
    comp = mc.quantization_compressor[fmt]
    want = {}
    for name, m in model.named_modules():
        scheme = getattr(m, "quantization_scheme", None)
        if scheme is None:
            continue
        args, w = scheme.weights, m.weight.data
        gs = None
        if args.strategy == "tensor_group":
            lo, hi = torch.aminmax(w)
            gs = generate_gparam(lo.reshape(1), hi.reshape(1))
            m.register_parameter("weight_global_scale", torch.nn.Parameter(gs, requires_grad=False))
            scale, zp = observe_weight_qparams(w, args, global_scale=gs)
        else:
            scale, zp = observe_weight_qparams(w, args)
        m.register_parameter("weight_scale", torch.nn.Parameter(scale, requires_grad=False))
        m.register_parameter("weight_zero_point", torch.nn.Parameter(zp, requires_grad=False))
        kw = dict(weight=w.clone(), scale=scale, zero_point=zp, quantization_args=args)
        if gs is not None:
            kw["global_scale"] = gs
        want[name] = comp.compress_weight(**kw)
    assert len(want) == 40
    mc.compress_model(model)
    for name, single in want.items():
        m = model.get_submodule(name)
        for key, value in single.items():
            assert_bit_equal(getattr(m, key).data, value.cpu(), f"{name}.{key}")
    held = {name: {k: p.data for k, p in model.get_submodule(name)._parameters.items() if p is not None}
            for name in want}
    mc.decompress_model(model)
    for name, data in held.items():
        m = model.get_submodule(name)
        single = comp.decompress_weight(compressed_data=data, quantization_args=m.quantization_scheme.weights)
        assert_bit_equal(m.weight.data, single.cpu(), f"{name} decompressed")
        assert m.weight.dtype == single.dtype


def test_wrapped_forward_and_in_place_weight_compression(gpu):
    """a module under apply_quantization_config: forward fake-quantizes the input (dynamic per
    token), the weight (put back afterwards) and the output as the scheme says (forward.py:355-412),
    bit for bit what fake_quantize gives on the same tensors; compress_quantized_weights leaves
    the oracle's int8 codes in the weight (compressed.py:33-73)"""
    from compressed_tensors_amd.quantization import (
        QuantizationArgs, QuantizationConfig, QuantizationScheme, apply_quantization_config,
        compress_quantized_weights, fake_quantize, observe_weight_qparams)
    from compressed_tensors_amd.quantization.helpers import compute_dynamic_scales_and_zp
    from oracle import quant as oq

    announce("wrapped forward")
    torch.manual_seed(3)
    w_spec = dict(num_bits=4, type="int", strategy="group", group_size=16, symmetric=False)
    i_spec = dict(num_bits=8, type="int", strategy="token", dynamic=True, symmetric=True)
    o_spec = dict(num_bits=8, type="float", strategy="tensor", dynamic=False, symmetric=True)
    scheme = QuantizationScheme(targets=["Linear"], weights=QuantizationArgs(**w_spec),
                                input_activations=QuantizationArgs(**i_spec),
                                output_activations=QuantizationArgs(**o_spec))
    model = torch.nn.Sequential(torch.nn.Linear(64, 32, bias=True)).to(torch.bfloat16).to(gpu)
    apply_quantization_config(model, QuantizationConfig(config_groups={"g": scheme}, quantization_status="frozen"))
    lin = model[0]
    w = lin.weight.data.clone()
    scale, zp = observe_weight_qparams(w, scheme.weights)
    lin.weight_scale.data.copy_(scale)
    lin.weight_zero_point.data.copy_(zp)
    lin.output_scale.data.fill_(0.01)
    x = torch.randn(2, 5, 64, device=gpu).bfloat16()
    got = model(x)
    s, z = compute_dynamic_scales_and_zp(x, scheme.input_activations)
    xq = fake_quantize(x, s, z, scheme.input_activations)
    wq = fake_quantize(w, scale, zp, scheme.weights)
    out = torch.nn.functional.linear(xq, wq, lin.bias)
    want = fake_quantize(out, lin.output_scale.data, lin.output_zero_point.data, scheme.output_activations)
    assert_bit_equal(got, want.cpu(), "forward")
    assert_bit_equal(lin.weight.data, w.cpu(), "the weight is put back")
    # the pieces against the oracle
    assert_bit_equal(wq, oq.fake_quantize(w.cpu(), scale.cpu(), zp.cpu(), oq._Args(**w_spec)), "weight on the grid")
    # calibration of a static output scheme leaves the output alone
    lin.quantization_status = "calibration"
    assert_bit_equal(model(x), out.cpu(), "calibration")
    lin.quantization_status = "frozen"
    lin.quantization_enabled = False
    assert_bit_equal(model(x), torch.nn.functional.linear(x, w, lin.bias).cpu(), "disabled")
    lin.quantization_enabled = True
    model.apply(compress_quantized_weights)
    assert lin.weight.dtype == torch.int8 and not lin.weight.requires_grad
    assert str(getattr(lin.quantization_status, "value", lin.quantization_status)) == "compressed"
    assert_bit_equal(lin.weight.data, oq.quantize(w.cpu(), scale.cpu(), zp.cpu(), oq._Args(**w_spec), dtype=torch.int8),
                     "int8 codes")
    model.apply(compress_quantized_weights)  # a second time changes nothing
    assert lin.weight.dtype == torch.int8
