"""Attention / KV-cache hooks (reference: src/compressed_tensors/modeling/, tests/test_modeling/).
CPU tests cover the plumbing on a tiny randomly initialised Llama; the GPU tests push
queries, keys and values through forward_quantize on the device."""
import json
from pathlib import Path

import pytest
import torch

from gpu_util import announce, assert_bit_equal
from oracle import quant as oq

GOLDEN = Path(__file__).parent / "golden"


def _tiny_llama(dtype=torch.float32):
    transformers = pytest.importorskip("transformers")
    config = transformers.LlamaConfig(
        hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
        num_key_value_heads=2, vocab_size=96, max_position_embeddings=64)
    torch.manual_seed(0)
    return transformers.LlamaForCausalLM(config).to(dtype).eval()


def _attention_modules(model):
    return [m for m in model.modules() if m.__class__.__name__.lower().endswith("attention")]


def test_hooked_attention_is_transparent_without_a_scheme():
    from compressed_tensors_amd.modeling import (
        IMPL_ATTR, KV_CACHE_ATTR, QuantizedAttentionImpl, QuantizedKVCache, initialize_hooked_attention,
        register_key_hook, register_query_hook, register_value_hook,
    )
    from compressed_tensors_amd.utils import InternalModule

    model = _tiny_llama()
    ids = torch.arange(10).reshape(1, 10) % 96
    with torch.no_grad():
        want = model(ids).logits
    seen = {}
    for attn in _attention_modules(model):
        initialize_hooked_attention(model, attn)
        initialize_hooked_attention(model, attn)  # a second call changes nothing
        assert isinstance(getattr(attn, IMPL_ATTR), QuantizedAttentionImpl)
        assert isinstance(getattr(attn, KV_CACHE_ATTR), QuantizedKVCache)
        assert isinstance(getattr(attn, IMPL_ATTR), InternalModule)
    assert model.config._attn_implementation == "ct_hooked_attention"
    attn = _attention_modules(model)[0]
    handles = [
        register_query_hook(attn, lambda m, q: seen.__setitem__("q", tuple(q.shape))),
        register_key_hook(attn, lambda m, k: seen.__setitem__("k", tuple(k.shape))),
        register_value_hook(attn, lambda m, v: seen.__setitem__("v", tuple(v.shape))),
    ]
    with torch.no_grad():
        got = model(ids).logits
    assert torch.equal(got, want)
    assert seen == {"q": (1, 4, 10, 16), "k": (1, 2, 10, 16), "v": (1, 2, 10, 16)}
    for h in handles:
        h.remove()
    # a hook that returns a tensor replaces the argument
    register_value_hook(attn, lambda m, v: torch.zeros_like(v))
    with torch.no_grad():
        assert not torch.equal(model(ids).logits, want)
    # generation goes through the real cache behind the wrapper
    with torch.no_grad():
        out = model.generate(ids, max_new_tokens=3, do_sample=False)
    assert out.shape == (1, 13)


def test_attention_qparams_and_scheme_checks():
    from compressed_tensors_amd.modeling import initialize_hooked_attention
    from compressed_tensors_amd.quantization import (
        QuantizationArgs, QuantizationScheme, initialize_module_for_quantization,
    )

    model = _tiny_llama(torch.bfloat16)
    attn = _attention_modules(model)[0]
    acts = QuantizationArgs(num_bits=8, type="float", symmetric=True, strategy="tensor")
    with pytest.raises(ValueError, match="no impl or kv_cache"):
        initialize_module_for_quantization(attn, QuantizationScheme(targets=[], input_activations=acts))
    initialize_hooked_attention(model, attn)
    initialize_module_for_quantization(attn, QuantizationScheme(targets=[], input_activations=acts))
    for base in "qkv":
        assert getattr(attn, f"{base}_scale").shape == (1,)
        assert getattr(attn, f"{base}_scale").dtype == torch.bfloat16
        assert getattr(attn, f"{base}_zero_point").dtype == torch.float8_e4m3fn
    per_head = QuantizationArgs(num_bits=8, type="float", symmetric=True, strategy="attn_head")
    initialize_module_for_quantization(attn, QuantizationScheme(targets=[], input_activations=per_head),
                                       force_zero_point=False)
    assert attn.q_scale.shape == (4, 1, 1) and attn.k_scale.shape == (2, 1, 1) and attn.v_scale.shape == (2, 1, 1)
    assert not hasattr(attn, "q_zero_point")
    weights = QuantizationArgs(num_bits=4, type="int", symmetric=True, strategy="channel")
    with pytest.raises(ValueError, match="weight quantization to attention"):
        initialize_module_for_quantization(attn, QuantizationScheme(targets=[], weights=weights,
                                                                    input_activations=acts))
    with pytest.raises(ValueError, match="without specifying input activations"):
        initialize_module_for_quantization(attn, QuantizationScheme(targets=[]))
    with pytest.raises(ValueError, match="output quantization to attention"):
        initialize_module_for_quantization(attn, QuantizationScheme(targets=[], input_activations=acts,
                                                                    output_activations=acts))


def test_config_helpers():
    from types import SimpleNamespace

    from compressed_tensors_amd.utils import get_head_dim, get_num_attn_heads, get_num_kv_heads, getattr_chain

    cfg = SimpleNamespace(hidden_size=64, head_dim=16)
    assert get_num_attn_heads(cfg) == 4 and get_head_dim(cfg) == 16
    assert get_head_dim(SimpleNamespace(hidden_size=64, num_attention_heads=8)) == 8
    with pytest.raises(ValueError):
        get_num_kv_heads(cfg)
    with pytest.raises(ValueError):
        get_head_dim(SimpleNamespace())
    obj = SimpleNamespace(a=SimpleNamespace(b=3))
    assert getattr_chain(obj, "a.b") == 3 and getattr_chain(obj, "a.c", None) is None
    with pytest.raises(AttributeError):
        getattr_chain(obj, "a.c")


class MockAttention(torch.nn.Module):
    pass


@pytest.mark.gpu
def test_static_attention_golden_on_gpu(gpu):
    """the reference's known answers for keys quantized per tensor and per head
    (test_static_lifecycle.py:278-386), through initialize_qparams and forward_quantize"""
    from compressed_tensors_amd.config import QuantizationStatus
    from compressed_tensors_amd.quantization import (
        QuantizationArgs, QuantizationScheme, calculate_qparams, forward_quantize, initialize_qparams,
    )

    gold = json.loads((GOLDEN / "static_lifecycle.json").read_text())
    x = torch.arange(24, dtype=torch.bfloat16).reshape(1, 2, 3, 4)
    for case in gold["attention_cases"]:
        announce("attention golden", case["args"])
        args = QuantizationArgs(**case["args"])
        attention = MockAttention().to(gpu)
        initialize_qparams(attention, "k", args, (2, None, 4), torch.bfloat16)
        attention.quantization_scheme = QuantizationScheme(targets=[], input_activations=args)
        attention.quantization_status = QuantizationStatus.INITIALIZED
        if args.strategy == "tensor":
            mn, mx = torch.aminmax(x)
            mn, mx = mn.reshape(1), mx.reshape(1)
        else:
            mn = torch.amin(x, dim=(0, 2, 3)).reshape(2, 1, 1)
            mx = torch.amax(x, dim=(0, 2, 3)).reshape(2, 1, 1)
        scale, zp = calculate_qparams(mn.to(gpu), mx.to(gpu), args)
        assert scale.shape == attention.k_scale.shape
        attention.k_scale.data = scale
        attention.k_zero_point.data = zp
        out = forward_quantize(attention, x.to(gpu), "k", args)
        o_scale, o_zp = oq.calculate_qparams(mn, mx, oq._Args(**case["args"]))
        assert_bit_equal(out, oq.fake_quantize(x, o_scale, o_zp, oq._Args(**case["args"])), "qdq")
        assert torch.allclose(out.cpu(), torch.tensor(case["qdq"]).to(out.dtype))
        assert torch.nn.functional.mse_loss(out.cpu().float(), x.float()) <= case["max_mse"]


@pytest.mark.gpu
@pytest.mark.parametrize("strategy", ["tensor", "attn_head"])
def test_hooked_attention_quantizes_q_k_v_on_gpu(strategy, gpu):
    """a tiny Llama with fp8 attention quantization: what reaches the attention function and
    the cache is forward_quantize of what the hooks saw, bit for bit against the oracle"""
    from compressed_tensors_amd.modeling import (
        IMPL_ATTR, KV_CACHE_ATTR, initialize_hooked_attention, register_key_hook, register_query_hook,
        register_value_hook,
    )
    from compressed_tensors_amd.quantization import (
        QuantizationArgs, QuantizationScheme, initialize_module_for_quantization,
    )

    announce("hooked attention", strategy)
    model = _tiny_llama(torch.bfloat16).to(gpu)
    ids = (torch.arange(12).reshape(1, 12) % 96).to(gpu)
    with torch.no_grad():
        plain = model(ids).logits
    spec = dict(num_bits=8, type="float", symmetric=True, strategy=strategy)
    args = QuantizationArgs(**spec)
    seen, passed_on = {}, {}
    for attn in _attention_modules(model):
        initialize_hooked_attention(model, attn)
        initialize_module_for_quantization(attn, QuantizationScheme(targets=[], input_activations=args))
        for base, heads in (("q", 4), ("k", 2), ("v", 2)):
            shape = getattr(attn, f"{base}_scale").shape
            assert shape == ((1,) if strategy == "tensor" else (heads, 1, 1))
            g = torch.Generator().manual_seed(heads)
            getattr(attn, f"{base}_scale").data = (torch.rand(shape, generator=g) * 0.01 + 0.004).bfloat16().to(gpu)
    attn = _attention_modules(model)[0]
    register_query_hook(attn, lambda m, q: seen.__setitem__("q", q.detach().clone()))
    register_key_hook(attn, lambda m, k: seen.__setitem__("k", k.detach().clone()))
    register_value_hook(attn, lambda m, v: seen.__setitem__("v", v.detach().clone()))
    # what the wrappers hand on: the cache's return value and the impl's query
    cache = getattr(attn, KV_CACHE_ATTR)
    cache.register_forward_hook(lambda m, a, out: passed_on.update(k=out[0].detach().clone(), v=out[1].detach().clone()))
    import transformers

    fn = transformers.modeling_utils.ALL_ATTENTION_FUNCTIONS
    original = fn[getattr(attn, IMPL_ATTR)._original_impl]

    def spy(module, query, *a, **kw):
        if module is attn:
            passed_on["q"] = query.detach().clone()
        return original(module, query, *a, **kw)

    fn.register(getattr(attn, IMPL_ATTR)._original_impl, spy)
    try:
        with torch.no_grad():
            quantized = model(ids).logits
    finally:
        fn.register(getattr(attn, IMPL_ATTR)._original_impl, original)
    assert not torch.equal(quantized, plain)
    for base in "qkv":
        scale = getattr(attn, f"{base}_scale").cpu()
        zp = getattr(attn, f"{base}_zero_point").cpu()
        want = oq.fake_quantize(seen[base].cpu(), scale, zp, oq._Args(**spec))
        assert_bit_equal(passed_on[base], want, f"{base} after the hook")
    # quantization switched off: back to the plain model
    for a in _attention_modules(model):
        a.quantization_enabled = False
    with torch.no_grad():
        assert torch.equal(model(ids).logits, plain)
