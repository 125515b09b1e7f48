"""Key / value quantization on the way into the KV cache
(reference: src/compressed_tensors/modeling/kvcache.py)."""
import inspect
import weakref
from typing import Callable, Optional, Tuple

from torch import Tensor
from torch.nn import Module
from torch.utils.hooks import RemovableHandle

from ..quantization.forward import forward_quantize
from ..utils.internal import InternalModule
from ._hooks import active_args, rewrite_argument

__all__ = ["KV_CACHE_ATTR", "QuantizedKVCache", "initialize_hooked_kv_cache",
           "register_key_hook", "register_value_hook"]

KV_CACHE_ATTR = "kv_cache"


class QuantizedKVCache(InternalModule):
    """Stands in for the `past_key_values` argument of an attention module: `update`
    fake-quantizes the new keys and values with the module's `k_*` / `v_*` parameters
    and passes them on to the cache it replaced, if there was one (kvcache.py:41-96).
    Being a module, it can carry forward hooks (transforms, calibration)."""

    def __init__(self, config, attn_module: Module):
        super().__init__()
        self.config = config
        self.attn_module = weakref.ref(attn_module)  # no reference cycle through the parent
        self.past_key_values = None

    def update(self, *args, **kwargs) -> Tuple[Tensor, Tensor]:
        return self(*args, **kwargs)

    def forward(self, key_states: Tensor, value_states: Tensor, *args, **kwargs) -> Tuple[Tensor, Tensor]:
        module = self.attn_module()
        quant_args = active_args(module)
        if quant_args is not None:
            key_states = forward_quantize(module, key_states, "k", quant_args)
            value_states = forward_quantize(module, value_states, "v", quant_args)
        cache = self.past_key_values() if self.past_key_values is not None else None
        self.past_key_values = None
        if cache is None:
            return key_states, value_states
        return cache.update(key_states, value_states, *args, **kwargs)

    def add_past_key_values(self, past_key_values) -> None:
        self.past_key_values = weakref.ref(past_key_values) if past_key_values is not None else None


def _swap_in_cache(module: Module, args, kwargs):
    """forward pre-hook of the attention module: its cache argument becomes the
    QuantizedKVCache, which remembers the real one for this call (kvcache.py:102-124)"""
    name = ("past_key_values" if "past_key_values" in inspect.signature(module.forward).parameters
            else "past_key_value")
    cache: QuantizedKVCache = getattr(module, KV_CACHE_ATTR)
    cache.add_past_key_values(kwargs.get(name))
    kwargs[name] = cache
    return args, kwargs


def initialize_hooked_kv_cache(model, module: Module) -> None:
    """attach a QuantizedKVCache to an attention module, once (kvcache.py:127-137)"""
    if hasattr(module, KV_CACHE_ATTR):
        return
    module.register_module(KV_CACHE_ATTR, QuantizedKVCache(model.config, module))
    module.register_forward_pre_hook(_swap_in_cache, with_kwargs=True)


def register_key_hook(module: Module, hook: Callable[[Module, Tensor], Optional[Tensor]]) -> RemovableHandle:
    """hook(module, keys after rope) -> replacement or None (kvcache.py:143-163)"""
    return rewrite_argument(getattr(module, KV_CACHE_ATTR), module, "key_states", hook)


def register_value_hook(module: Module, hook: Callable[[Module, Tensor], Optional[Tensor]]) -> RemovableHandle:
    """hook(module, values) -> replacement or None (kvcache.py:166-183)"""
    return rewrite_argument(getattr(module, KV_CACHE_ATTR), module, "value_states", hook)
