"""Which modules and parameters of a model a list of targets names (reference:
src/compressed_tensors/utils/match.py).  A target is a module's dotted name, a regular
expression over it behind the prefix "re:", or the name of a class the module derives from.
Modules this library adds to a model (InternalModule) never match."""
import logging
import re
from typing import Dict, Iterable, Iterator, List, Optional, Tuple, Union

import torch

from .internal import InternalModule

__all__ = ["match_named_modules", "match_named_parameters", "match_modules_set", "is_match",
           "is_narrow_match", "match_targets"]

_LOGGER = logging.getLogger(__name__)
Fused = Dict[str, Iterable[str]]


def _as_list(entries) -> List[str]:
    if entries is None:
        return []
    return [entries] if isinstance(entries, str) else list(entries)


def _name_matches(name: str, target: str, fused: Optional[Fused] = None) -> bool:
    """match.py:287-312: equality, or a regular expression matched from the start of the
    name.  `fused` maps the suffix of a fused module ("qkv_proj") to the suffixes of the
    modules it stands for: the fused module matches where any of those would."""
    if fused:
        for suffix, shards in fused.items():
            if name.endswith(suffix):
                stem = name[: len(name) - len(suffix)]
                return any(_name_matches(stem + shard, target) for shard in shards)
    if target.startswith("re:"):
        return re.match(target[3:], name) is not None
    return name == target


_CLASS_NAMES: Dict[type, frozenset] = {}


def _class_matches(module: torch.nn.Module, target: str) -> bool:
    """match.py:315-336: any torch module class among the module's bases carries the name
    (vLLM's LinearBase counts as Linear)"""
    names = _CLASS_NAMES.get(type(module))
    if names is None:
        found = {c.__name__ for c in type(module).__mro__ if issubclass(c, torch.nn.Module)}
        if "LinearBase" in found:
            found.add("Linear")
        names = _CLASS_NAMES[type(module)] = frozenset(found)
    return target in names


def _one(name: str, module: torch.nn.Module, target: str, fused: Optional[Fused]) -> bool:
    return _name_matches(name, target, fused) or _class_matches(module, target)


def is_match(name: str, module: torch.nn.Module, targets: Union[str, Iterable[str]],
             ignore: Union[str, Iterable[str], None] = (), fused: Optional[Fused] = None) -> bool:
    """match.py:214-257"""
    if isinstance(module, InternalModule):
        return False
    if not any(_one(name, module, t, fused) for t in _as_list(targets)):
        return False
    return not any(_one(name, module, t, fused) for t in _as_list(ignore))


def match_targets(name: str, module: torch.nn.Module, targets: Optional[Iterable[str]]) -> List[str]:
    """the targets that name this module, most specific first: exact names, then regular
    expressions, then class names (match.py:122-157; configurations are merged in this order)"""
    if isinstance(module, InternalModule):
        return []
    ordered = sorted(_as_list(targets), key=lambda t: ("re:" in t, t))
    hits = [t for t in ordered if _name_matches(name, t)]
    hits += [t for t in ordered if t not in hits and _class_matches(module, t)]
    return hits


def match_named_modules(model: torch.nn.Module, targets: Optional[Iterable[str]],
                        ignore: Optional[Iterable[str]] = None, fused: Optional[Fused] = None,
                        warn_on_fail: bool = False) -> Iterator[Tuple[str, torch.nn.Module]]:
    """(name, module) in the order of model.named_modules() for every module a target names
    and no ignore entry does (match.py:39-75)"""
    targets, ignore = _as_list(targets), _as_list(ignore)
    unmatched = set(targets)
    for name, module in model.named_modules():
        if isinstance(module, InternalModule):
            continue
        if warn_on_fail and unmatched:  # every target that names the module has found one
            unmatched.difference_update([t for t in unmatched if _one(name, module, t, fused)])
        if not any(_one(name, module, t, fused) for t in targets):
            continue
        if not any(_one(name, module, t, fused) for t in ignore):
            yield name, module
    if warn_on_fail:
        for t in unmatched:
            _LOGGER.warning("Could not match `%s` in instance of %s", t, type(model).__name__)


def match_named_parameters(model: torch.nn.Module, targets: Optional[Iterable[str]],
                           ignore: Optional[Iterable[str]] = None, fused: Optional[Fused] = None,
                           warn_on_fail: bool = False
                           ) -> Iterator[Tuple[str, torch.nn.Module, torch.nn.Parameter]]:
    """(full name, owning module, parameter) for every parameter whose dotted name a target
    names and no ignore entry does (match.py:78-123)"""
    targets, ignore = _as_list(targets), _as_list(ignore)
    unmatched = set(targets)
    for mod_name, module in model.named_modules():
        if isinstance(module, InternalModule):
            continue
        for p_name, param in module.named_parameters(recurse=False):
            full = f"{mod_name}.{p_name}"
            for t in targets:  # once per target that names it, as the reference yields
                if _name_matches(full, t, fused):
                    unmatched.discard(t)
                    if not any(_name_matches(full, i, fused) for i in ignore):
                        yield full, module, param
    if warn_on_fail:
        for t in unmatched:
            _LOGGER.warning("Could not match `%s` in instance of %s", t, type(model).__name__)


def match_modules_set(model: torch.nn.Module, targets: Optional[Iterable[str]],
                      ignore: Optional[Iterable[str]] = None) -> Iterator[List[torch.nn.Module]]:
    """modules in groups shaped like `targets`: walking the model, a group is given out as soon
    as every target has met one module (the q, k and v projections of one layer, a norm with
    the projections behind it); a target met twice before that is an error (match.py:160-211)"""
    targets, ignore = _as_list(targets), _as_list(ignore)
    found: Dict[str, Optional[torch.nn.Module]] = dict.fromkeys(targets)
    for name, module in model.named_modules():
        for t in targets:
            if is_match(name, module, t, ignore):
                if found[t] is not None:
                    raise ValueError(f"Matched a {t} twice before completing set")
                found[t] = module
        if targets and all(m is not None for m in found.values()):
            yield [found[t] for t in targets]
            found = dict.fromkeys(targets)
    left_over = [t for t, m in found.items() if m is not None]  # met, but their set never filled
    if left_over:
        raise ValueError(f"Unable to match targets into set: {left_over}")


def is_narrow_match(model: torch.nn.Module, targets: Union[str, Iterable[str]], name: str,
                    module: Optional[torch.nn.Module] = None) -> bool:
    """a target names the module but not the module's parent (match.py:260-284)"""
    module = module if module is not None else model.get_submodule(name)
    parent_name = name.rsplit(".", 1)[0]
    parent = model.get_submodule(parent_name)
    return any(is_match(name, module, t) and not is_match(parent_name, parent, t)
               for t in _as_list(targets))
