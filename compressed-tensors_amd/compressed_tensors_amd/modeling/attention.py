"""Query quantization in front of the attention function
(reference: src/compressed_tensors/modeling/attention.py)."""
from typing import Callable, Optional

from torch import Tensor
from torch.nn import Module
from torch.utils.hooks import RemovableHandle

from ..quantization.forward import forward_quantize
from ..utils.internal import InternalModule
from ._hooks import active_args, rewrite_argument
from .kvcache import initialize_hooked_kv_cache

__all__ = ["IMPL_ATTR", "QuantizedAttentionImpl", "initialize_hooked_attention", "register_query_hook"]

IMPL_ATTR = "impl"
HOOKED_ATTENTION_NAME = "ct_hooked_attention"


def _attention_functions():
    from transformers.masking_utils import ALL_MASK_ATTENTION_FUNCTIONS
    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS

    return ALL_ATTENTION_FUNCTIONS, ALL_MASK_ATTENTION_FUNCTIONS


class QuantizedAttentionImpl(InternalModule):
    """The attention function as a module: fake-quantizes the queries with the parent's
    `q_*` parameters, then calls the implementation the model was using before
    (attention.py:43-89).  Being a module, it can carry forward hooks."""

    _original_impl = "eager"

    def __init__(self, config):
        super().__init__()
        self.config = config

    def forward(self, module: Module, query: Tensor, key: Tensor, value: Tensor, *args, **kwargs):
        quant_args = active_args(module)
        if quant_args is not None:
            query = forward_quantize(module, query, "q", quant_args)
        functions, _ = _attention_functions()
        return functions[QuantizedAttentionImpl._original_impl](module, query, key, value, *args, **kwargs)


def _hooked_attention(module: Module, *args, **kwargs):
    impl = getattr(module, IMPL_ATTR, None)
    assert impl is not None, (
        f"Using {HOOKED_ATTENTION_NAME} attention implementation, "
        f"but attention module does not have {IMPL_ATTR} submodule.")
    return impl(module, *args, **kwargs)


def initialize_hooked_attention(model, module: Module) -> None:
    """attach a QuantizedAttentionImpl and a QuantizedKVCache to an attention module and
    make the model call attention through them; one model at a time (attention.py:105-127)"""
    if not hasattr(module, IMPL_ATTR):
        module.register_module(IMPL_ATTR, QuantizedAttentionImpl(model.config))
    current = model.config._attn_implementation
    if current != HOOKED_ATTENTION_NAME:
        functions, masks = _attention_functions()
        QuantizedAttentionImpl._original_impl = current
        functions.register(HOOKED_ATTENTION_NAME, _hooked_attention)
        masks.register(HOOKED_ATTENTION_NAME, masks[current])
        model.set_attn_implementation(HOOKED_ATTENTION_NAME)
        assert model.config._attn_implementation == HOOKED_ATTENTION_NAME
    initialize_hooked_kv_cache(model, module)


def register_query_hook(module: Module, hook: Callable[[Module, Tensor], Optional[Tensor]]) -> RemovableHandle:
    """hook(module, queries after rope) -> replacement or None (attention.py:133-147)"""
    return rewrite_argument(getattr(module, IMPL_ATTR), module, "query", hook)
