"""Bitmask packing and small tensor utilities.

pack_bitmasks / unpack_bitmasks reproduce numpy.packbits / unpackbits with
bitorder="little" (reference: utils/helpers.py:302-339) on the GPU; shard /
combine helpers mirror utils/helpers.py:237-299; merge_names mirrors
utils/safetensors_load.py:115-125.
"""
import contextlib
import warnings
from functools import wraps
from typing import Any, Callable, Dict, List, Optional

import torch

from compressed_tensors_amd import _lib

__all__ = [
    "pack_bitmasks",
    "unpack_bitmasks",
    "shard_tensor",
    "combine_shards",
    "merge_names",
    "tensor_follows_mask_structure",
    "split_param_name",
    "nest_state_dict",
    "load_safetensors_state_dict",
    "getattr_chain",
    "get_num_attn_heads",
    "get_num_kv_heads",
    "get_head_dim",
    "Aliasable",
    "ParameterizedDefaultDict",
    "patch_attr",
    "deprecated",
    "replace_module",
    "fix_fsdp_module_name",
    "is_compressed_tensors_config",
    "infer_compressor_from_model_config",
]


def pack_bitmasks(bytemasks: torch.Tensor) -> torch.Tensor:
    """[..., C] bool -> [..., ceil(C/8)] uint8, bit j of byte k = column 8k+j."""
    _lib.require_gpu(bytemasks)
    m = bytemasks.contiguous()
    if m.dtype not in (torch.bool, torch.uint8, torch.int8):
        m = m != 0
    cols = m.shape[-1]
    rows = m.numel() // cols if cols else 0
    out = torch.empty(tuple(m.shape[:-1]) + ((cols + 7) // 8,), dtype=torch.uint8, device=m.device)
    _lib.check(
        _lib.load().ctmi_pack_bitmasks(m.data_ptr(), out.data_ptr(), rows, cols,
                                       _lib.stream_of(m.device))
    )
    return out


def unpack_bitmasks(packed_bitmasks: torch.Tensor, original_shape: List[int]) -> torch.Tensor:
    """inverse of pack_bitmasks; returns a bool tensor of `original_shape`"""
    _lib.require_gpu(packed_bitmasks)
    p = packed_bitmasks.contiguous()
    shape = [int(d) for d in original_shape]
    cols = shape[-1]
    rows = 1
    for d in shape[:-1]:
        rows *= d
    if p.numel() != rows * ((cols + 7) // 8):
        raise ValueError(
            f"cannot reshape {p.numel()} bitmask bytes into shape {shape}"
        )
    out = torch.empty(shape, dtype=torch.bool, device=p.device)
    _lib.check(
        _lib.load().ctmi_unpack_bitmasks(p.data_ptr(), out.data_ptr(), rows, cols,
                                         _lib.stream_of(p.device))
    )
    return out


def shard_tensor(tensor: torch.Tensor, shard_sizes: List[int], dim: int = 0) -> List[torch.Tensor]:
    if sum(shard_sizes) != tensor.size(dim):
        raise ValueError(
            "Sum of shard_sizes must equal the size of the tensor along the specified dimension."
        )
    out, start = [], 0
    for size in shard_sizes:
        out.append(tensor.narrow(dim, start, size))
        start += size
    return out


def combine_shards(shards, dim=0):
    if not shards:
        raise ValueError("The list of shards is empty.")
    if len({s.dtype for s in shards}) > 1:
        raise ValueError("All shards must have the same dtype.")
    return torch.cat(list(shards), dim=dim)


def merge_names(parent_name: str, child_name: str) -> str:
    if not parent_name:
        return child_name
    if not child_name:
        return parent_name
    return parent_name + "." + child_name


def tensor_follows_mask_structure(tensor: torch.Tensor, mask: str = "2:4") -> bool:
    n, m = (int(p) for p in mask.split(":"))
    zero_counts = (tensor.reshape(-1, m) == 0).sum(dim=1)
    if not bool(torch.all(zero_counts >= n)):
        raise ValueError()
    return True


def split_param_name(full_name: str, param_name: str):
    """'a.b.<param_name>' -> 'a.b'; None when full_name does not end in '.<param_name>'"""
    suffix = "." + param_name
    if full_name.endswith(suffix) and len(full_name) > len(suffix):
        return full_name[: -len(suffix)]
    return None


def nest_state_dict(state_dict, params_to_nest, return_unmatched_params: bool = False):
    """Group compression parameters by owning module:
    {module_path: {param_name: tensor}} (+ the entries that matched nothing).
    Reference: utils/safetensors_load.py:251-291."""
    nested, unmatched = {}, {}
    names = set(params_to_nest)
    if not any("." in n for n in names):
        # every name is a last component: one split per key
        for key, value in state_dict.items():
            module_path, _, last = key.rpartition(".")
            if module_path and last in names:
                nested.setdefault(module_path, {})[last] = value
            else:
                unmatched[key] = value
        return (nested, unmatched) if return_unmatched_params else nested
    for key, value in state_dict.items():
        hit = False
        for param_name in params_to_nest:
            module_path = split_param_name(key, param_name)
            if module_path:
                nested.setdefault(module_path, {})[param_name] = value
                hit = True
        if not hit:
            unmatched[key] = value
    return (nested, unmatched) if return_unmatched_params else nested


def load_safetensors_state_dict(path, device="cpu"):
    """All tensors of a .safetensors file, or of every such file in a directory."""
    import os

    from safetensors import safe_open

    path = str(path)
    files = (
        sorted(os.path.join(path, f) for f in os.listdir(path) if f.endswith(".safetensors"))
        if os.path.isdir(path)
        else [path]
    )
    out = {}
    for f in files:
        with safe_open(f, framework="pt", device=str(device)) as fh:
            for k in fh.keys():
                out[k] = fh.get_tensor(k)
    return out


_MISSING = object()


def getattr_chain(obj, chain_str: str, default=_MISSING):
    """getattr along a dotted path; `default` (if given) when a link is missing
    (reference: utils/helpers.py:145-171)"""
    for name in chain_str.split("."):
        if not hasattr(obj, name):
            if default is _MISSING:
                raise AttributeError(f"{obj} object has no attribute {name}")
            return default
        obj = getattr(obj, name)
    return obj


def get_num_attn_heads(config) -> int:
    """reference: utils/helpers.py:404-422"""
    if hasattr(config, "num_attention_heads"):
        return config.num_attention_heads
    if hasattr(config, "hidden_size") and hasattr(config, "head_dim"):
        return config.hidden_size // config.head_dim
    raise ValueError("Cannot determine num_attention_heads from config. Config must define either "
                     f"`num_attention_heads` or both `hidden_size` and `head_dim`. {config}")


def get_num_kv_heads(config) -> int:
    """reference: utils/helpers.py:425-439"""
    if hasattr(config, "num_key_value_heads"):
        return config.num_key_value_heads
    raise ValueError("Cannot determine num_key_value_heads from config. Config must define "
                     f"`num_key_value_heads`. {config}")


def get_head_dim(config) -> int:
    """reference: utils/helpers.py:442-460"""
    if hasattr(config, "head_dim"):
        return config.head_dim
    if hasattr(config, "hidden_size") and hasattr(config, "num_attention_heads"):
        return config.hidden_size // config.num_attention_heads
    raise ValueError("Cannot determine head_dim from config. Config must define either `head_dim` "
                     f"or both `hidden_size` and `num_attention_heads`. {config}")


# ------------------------------------------------------------------ small host utilities
FSDP_WRAPPER_NAME = "_fsdp_wrapped_module"


def fix_fsdp_module_name(name: str) -> str:
    """a module name without FSDP's wrapper component, wherever it sits (utils/helpers.py:80-90)"""
    return name.replace(FSDP_WRAPPER_NAME + ".", "").replace("." + FSDP_WRAPPER_NAME, "")


def replace_module(model: torch.nn.Module, name: str, new_module: torch.nn.Module) -> None:
    """put `new_module` where the dotted `name` points (utils/helpers.py:118-127)"""
    parent_name, _, child = name.rpartition(".")
    parent = model.get_submodule(parent_name) if parent_name else model
    setattr(parent, child, new_module)


def is_compressed_tensors_config(compression_config: Any) -> bool:
    """is this transformers' CompressedTensorsConfig (False where transformers has none;
    utils/helpers.py:130-142)"""
    try:
        from transformers.utils.quantization_config import CompressedTensorsConfig
    except ImportError:
        return False
    return isinstance(compression_config, CompressedTensorsConfig)


def infer_compressor_from_model_config(pretrained_model_name_or_path: str):
    """the sparsity compressor a model's config.json names, or None (utils/helpers.py:56-77)"""
    from transformers import AutoConfig

    from compressed_tensors_amd.compressors import BaseCompressor, ModelCompressor
    from compressed_tensors_amd.config import SparsityCompressionConfig

    config = AutoConfig.from_pretrained(pretrained_model_name_or_path)
    sparsity = ModelCompressor.parse_sparsity_config(getattr(config, "quantization_config", None)
                                                     or getattr(config, "compression_config", None))
    if sparsity is None:
        return None
    fmt = sparsity.get("format")
    return BaseCompressor.load_from_registry(
        fmt, config=SparsityCompressionConfig.load_from_registry(fmt, **sparsity))


def deprecated(future_name: Optional[str] = None, message: Optional[str] = None) -> Callable:
    """decorator: calling the function warns (DeprecationWarning) that it will go, and what
    to call instead (utils/helpers.py:176-203)"""
    def decorator(func):
        text = message
        if text is None:
            text = f"{func.__name__} is deprecated and will be removed in a future release"
            if future_name is not None:
                text += f". Please use {future_name} instead."

        @wraps(func)
        def wrapped(*args, **kwargs):
            warnings.warn(text, DeprecationWarning, stacklevel=2)
            return func(*args, **kwargs)

        return wrapped

    return decorator


class Aliasable:
    """mixin for enums some of whose members are other names for a member: equality and
    hashing go by the member an alias stands for (utils/helpers.py:206-234)"""

    @staticmethod
    def get_aliases() -> Dict[str, str]:
        raise NotImplementedError()

    def _canonical(self, value):
        return self.get_aliases().get(value, value)

    def __eq__(self, other):
        other_value = other.value if isinstance(other, type(self)) else other
        try:
            return self._canonical(self.value) == self._canonical(other_value)
        except TypeError:  # an unhashable `other` is no member
            return False

    def __ne__(self, other):
        return not self.__eq__(other)

    def __hash__(self):
        return hash(self._canonical(self.value))


@contextlib.contextmanager
def patch_attr(base: object, attr: str, value: Any):
    """`base.attr = value` inside the with block; afterwards the old value is back, or the
    attribute gone if there was none (utils/helpers.py:343-368)"""
    missing = object()
    before = getattr(base, attr, missing)
    setattr(base, attr, value)
    try:
        yield
    finally:
        if before is missing:
            delattr(base, attr)
        else:
            setattr(base, attr, before)


class ParameterizedDefaultDict(dict):
    """a defaultdict whose factory is given the missing key (a tuple key as its arguments)
    and, through get(), keyword arguments that are not part of the key
    (utils/helpers.py:371-401)"""

    def __init__(self, default_factory: Callable[..., Any]):
        super().__init__()
        self.default_factory = default_factory
        self._factory_kwargs: Dict[str, Any] = {}

    def __missing__(self, key: Any) -> Any:
        args = key if isinstance(key, tuple) else (key,)
        value = self[key] = self.default_factory(*args, **self._factory_kwargs)
        return value

    def get(self, *args, factory_kwargs: Optional[Dict[str, Any]] = None) -> Any:
        with patch_attr(self, "_factory_kwargs", dict(factory_kwargs or {})):
            return self[args]
