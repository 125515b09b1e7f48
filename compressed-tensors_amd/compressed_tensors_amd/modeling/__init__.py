"""Hooks that put `forward_quantize` on the queries, keys and values of an attention
module (reference: src/compressed_tensors/modeling/)."""
from .attention import (IMPL_ATTR, QuantizedAttentionImpl, initialize_hooked_attention,
                        register_query_hook)
from .kvcache import (KV_CACHE_ATTR, QuantizedKVCache, initialize_hooked_kv_cache,
                      register_key_hook, register_value_hook)

__all__ = [
    "IMPL_ATTR", "KV_CACHE_ATTR", "QuantizedAttentionImpl", "QuantizedKVCache",
    "initialize_hooked_attention", "initialize_hooked_kv_cache", "register_query_hook",
    "register_key_hook", "register_value_hook",
]
