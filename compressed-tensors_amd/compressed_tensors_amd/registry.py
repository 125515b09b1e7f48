"""String-keyed class registry used for compressor and transform plug-ins.

Same contract as the reference's RegistryMixin (registry/registry.py:68-200):
`@Base.register(name=..., alias=...)`, `Base.load_from_registry(name, **kw)`,
`Base.get_value_from_registry(name)`, `Base.registered_names()`; names are
normalised (lower case, `_` and space -> `-`).  Each root class that mixes this
in owns a separate table.
"""
from typing import Dict, List, Optional, Union

__all__ = ["RegistryMixin", "standardize_lookup_name"]


def standardize_lookup_name(name: str) -> str:
    return name.replace("_", "-").replace(" ", "-").lower()


class RegistryMixin:
    _ctmi_registry: Dict[str, type]
    _ctmi_aliases: Dict[str, str]

    @classmethod
    def _tables(cls):
        # the table lives on the first class in the MRO that mixes the registry in directly
        for base in cls.__mro__:
            if RegistryMixin in base.__bases__:
                if "_ctmi_registry" not in base.__dict__:
                    base._ctmi_registry = {}
                    base._ctmi_aliases = {}
                return base._ctmi_registry, base._ctmi_aliases
        raise TypeError(f"{cls} does not derive from RegistryMixin")

    @classmethod
    def register(cls, name: Optional[str] = None, alias: Union[List[str], str, None] = None):
        def decorator(value: type):
            cls.register_value(value, name=name, alias=alias)
            return value

        return decorator

    @classmethod
    def register_value(cls, value: type, name: Optional[str] = None, alias=None):
        registry, aliases = cls._tables()
        key = standardize_lookup_name(name or value.__name__)
        if not issubclass(value, cls):
            raise ValueError(f"{value} is not a subclass of {cls}")
        if key in registry and registry[key] is not value:
            raise RuntimeError(f"{key} is already registered as {registry[key]}")
        registry[key] = value
        if alias is not None:
            for a in [alias] if isinstance(alias, str) else alias:
                a = standardize_lookup_name(a)
                if a in aliases and aliases[a] != key:
                    raise KeyError(f"alias {a} already points to {aliases[a]}")
                aliases[a] = key

    @classmethod
    def get_value_from_registry(cls, name: str) -> type:
        registry, aliases = cls._tables()
        key = standardize_lookup_name(name)
        key = aliases.get(key, key)
        if key not in registry:
            raise KeyError(
                f"Unable to find {name} registered under type {cls.__name__}.\n"
                f"Registered values for {cls.__name__}: {sorted(registry)}"
            )
        return registry[key]

    @classmethod
    def load_from_registry(cls, name: str, **constructor_kwargs):
        return cls.get_value_from_registry(name)(**constructor_kwargs)

    @classmethod
    def registered_names(cls) -> List[str]:
        return list(cls._tables()[0])

    @classmethod
    def registered_aliases(cls) -> List[str]:
        return list(cls._tables()[1])
