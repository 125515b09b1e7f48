"""What the attention and cache wrappers share."""
import inspect
from typing import Callable, Optional

from torch import Tensor
from torch.nn import Module


def active_args(module: Module):
    """the activation arguments an attention module quantizes q / k / v with, or None
    (reference: modeling/attention.py:74-79, kvcache.py:71-77)"""
    scheme = getattr(module, "quantization_scheme", None)
    args = getattr(scheme, "input_activations", None)
    if args is None or not getattr(module, "quantization_enabled", True):
        return None
    return args


def rewrite_argument(wrapper: Module, owner: Module, name: str,
                     hook: Callable[[Module, Tensor], Optional[Tensor]]):
    """forward pre-hook on `wrapper` that shows argument `name` of its forward to
    hook(owner, tensor) and replaces it when the hook returns a tensor
    (reference: attention.py:125-146, kvcache.py:146-183)"""
    signature = inspect.signature(wrapper.forward)

    def pre(_, args, kwargs):
        bound = signature.bind(*args, **kwargs)
        replacement = hook(owner, bound.arguments[name])
        if replacement is not None:
            bound.arguments[name] = replacement
        return bound.args, bound.kwargs

    return wrapper.register_forward_pre_hook(pre, with_kwargs=True)
