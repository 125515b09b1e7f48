"""String-keyed registry for compressor, config and transform plug-ins.

The contract of the reference's registry (registry/registry.py): a table per class that
`register` is called on; names are normalised (lower case, `_` and space -> `-`); aliases;
`"/path/to/file.py:Name"` loads a value from a file; `registry_requires_subclass` on a class
makes it refuse values that do not derive from it.  On top of that a class here also finds
what was registered on the classes it derives from, nearest first.
"""
import importlib.util
from collections import defaultdict
from typing import Any, Dict, List, Optional, Union

__all__ = [
    "RegistryMixin",
    "register",
    "get_from_registry",
    "registered_names",
    "registered_aliases",
    "standardize_lookup_name",
]

_REGISTRY: Dict[type, Dict[str, Any]] = defaultdict(dict)
_ALIAS_REGISTRY: Dict[type, Dict[str, str]] = defaultdict(dict)


def standardize_lookup_name(name: str) -> str:
    """registry.py:40-54"""
    return name.replace("_", "-").replace(" ", "-").lower()


def _alias_list(alias: Union[None, str, List[str]]) -> List[str]:
    if alias is None:
        return []
    return [standardize_lookup_name(a) for a in ([alias] if isinstance(alias, str) else alias)]


def _validate_subclass(parent_class: type, child_class: type) -> None:
    if not (isinstance(child_class, type) and issubclass(child_class, parent_class)):
        raise ValueError(f"class {child_class} is not a subclass of the class it is "
                         f"registered for: {parent_class}.")


def register_alias(name: str, parent_class: type, alias: Union[str, List[str], None] = None) -> None:
    """the aliases, and the name itself, point to `name` (registry.py:300-332)"""
    names = _alias_list(alias)
    if name in names:
        raise KeyError(f"Attempting to register alias {name}, that is identical to the "
                       f"standardized name: {name}.")
    table = _ALIAS_REGISTRY[parent_class]
    for a in names + [name]:
        if a in table and table[a] != name:
            raise KeyError(f"Attempting to register alias {a} as {name} however {a} has "
                           f"already been registered as {table[a]}")
        table[a] = name


def register(parent_class: type, value: Any, name: Optional[str] = None,
             alias: Union[List[str], str, None] = None, require_subclass: bool = False) -> None:
    """registry.py:203-240; registering the same value under its name again is allowed"""
    key = standardize_lookup_name(name if name is not None else value.__name__)
    if require_subclass:
        _validate_subclass(parent_class, value)
    known = _REGISTRY[parent_class].get(key)
    if known is not None and known is not value:
        raise RuntimeError(f"Attempting to register name {key} as {value} however {key} has "
                           f"already been registered as {known}")
    register_alias(name=key, alias=alias, parent_class=parent_class)
    _REGISTRY[parent_class][key] = value


def _value_from_file(module_path: str, value_name: str) -> Any:
    """registry.py:335-353"""
    spec = importlib.util.spec_from_file_location(f"plugin_module_for_{value_name}", module_path)
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    value = getattr(module, value_name, None)
    if not value:
        raise RuntimeError(f"Unable to find attribute {value_name} in module {module_path}")
    return value


def _tables_of(parent_class: type):
    """the class's own table first, then those of its bases"""
    return [c for c in parent_class.__mro__ if c in _REGISTRY or c in _ALIAS_REGISTRY] or [parent_class]


def get_from_registry(parent_class: type, name: str, require_subclass: bool = False) -> Any:
    """registry.py:243-277"""
    if ":" in name:
        module_path, value_name = name.split(":")
        value = _value_from_file(module_path, value_name)
    else:
        key = standardize_lookup_name(name)
        value = None
        for owner in _tables_of(parent_class):
            value = _REGISTRY[owner].get(_ALIAS_REGISTRY[owner].get(key, key))
            if value is not None:
                break
        if value is None:
            raise KeyError(
                f"Unable to find {key} registered under type {parent_class}.\n"
                f"Registered values for {parent_class}: {registered_names(parent_class)}\n"
                f"Registered aliases for {parent_class}: {registered_aliases(parent_class)}")
    if require_subclass:
        _validate_subclass(parent_class, value)
    return value


def registered_names(parent_class: type) -> List[str]:
    """registry.py:280-285"""
    return [n for owner in _tables_of(parent_class) for n in _REGISTRY[owner]]


def registered_aliases(parent_class: type) -> List[str]:
    """aliases that are not names (registry.py:288-297)"""
    names = set(registered_names(parent_class))
    return [a for owner in _tables_of(parent_class) for a in _ALIAS_REGISTRY[owner] if a not in names]


class RegistryMixin:
    """`@Base.register(name=..., alias=...)`, `Base.load_from_registry(name, **kwargs)`,
    `Base.get_value_from_registry(name)`, `Base.registered_names()` (registry.py:68-200)"""

    # True in a class: values registered on it and fetched from it must derive from it
    registry_requires_subclass: bool = False

    @classmethod
    def register(cls, name: Optional[str] = None, alias: Union[List[str], str, None] = None):
        def decorator(value: Any):
            cls.register_value(value, name=name, alias=alias)
            return value

        return decorator

    @classmethod
    def register_value(cls, value: Any, name: Optional[str] = None,
                       alias: Union[List[str], str, None] = None) -> None:
        register(cls, value, name=name, alias=alias, require_subclass=cls.registry_requires_subclass)

    @classmethod
    def load_from_registry(cls, name: str, **constructor_kwargs):
        return cls.get_value_from_registry(name)(**constructor_kwargs)

    @classmethod
    def get_value_from_registry(cls, name: str):
        return get_from_registry(cls, name, require_subclass=cls.registry_requires_subclass)

    @classmethod
    def registered_names(cls) -> List[str]:
        return registered_names(cls)

    @classmethod
    def registered_aliases(cls) -> List[str]:
        return registered_aliases(cls)
