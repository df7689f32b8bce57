"""Name -> (class, config class) registries with config-driven construction.

Counterpart of the reference's optimus_dl/core/registry.py for the one registry
this path uses ("model_transform", optimus_dl/modules/model_transforms/__init__.py:7-9):
``make_registry(name)`` returns ``(table, register, build)``; ``register(name,
cfg_cls)`` decorates a class; ``build(cfg, **kwargs)`` looks up ``cfg["_name"]``,
overlays the user's keys on the defaults of the registered config class
(registry.py:528-531 in the reference) and calls ``cls(cfg, **kwargs)``.

No OmegaConf dependency: any mapping (dict, DictConfig, dataclass instance) is
accepted as the user config.
"""

from __future__ import annotations

import dataclasses
from collections.abc import Mapping
from dataclasses import dataclass
from typing import Any, Callable

_REGISTRIES: dict[str, dict[str, tuple[type, type | None]]] = {}


@dataclass
class RegistryConfigStrict:
    """Config base that only knows ``_name``; unknown keys are rejected at build time."""

    _name: str | None = None


@dataclass
class RegistryConfig(dict):
    """Open config base: declared fields are attributes, anything else rides along
    as dictionary items (so extra keys in a YAML file are tolerated)."""

    _name: str | None = None

    def __post_init__(self) -> None:  # dict part is filled by build()
        pass

    def __getattr__(self, key: str) -> Any:  # only reached when normal lookup fails
        try:
            return self[key]
        except KeyError:
            raise AttributeError(key) from None

    def __hash__(self):  # dict subclasses lose hashing; identity is enough here
        return id(self)


def _to_plain_dict(cfg: Any) -> dict[str, Any]:
    if cfg is None:
        return {}
    if dataclasses.is_dataclass(cfg) and not isinstance(cfg, type):
        out = {f.name: getattr(cfg, f.name) for f in dataclasses.fields(cfg)}
        if isinstance(cfg, Mapping):
            out.update({k: v for k, v in cfg.items()})
        return out
    if isinstance(cfg, Mapping):
        return {str(k): v for k, v in cfg.items()}
    if hasattr(cfg, "__dict__"):
        return dict(vars(cfg))
    raise TypeError(f"cannot read a config of type {type(cfg).__name__}")


def instantiate_config(cfg_cls: type | None, user: Mapping[str, Any]) -> Any:
    """Defaults of ``cfg_cls`` overlaid with ``user``; extra keys kept for open configs."""
    if cfg_cls is None:
        return dict(user)
    names = {f.name for f in dataclasses.fields(cfg_cls)}
    known = {k: v for k, v in user.items() if k in names}
    extra = {k: v for k, v in user.items() if k not in names}
    obj = cfg_cls(**known)
    if extra:
        if isinstance(obj, dict):
            obj.update(extra)
        else:
            raise ValueError(f"{cfg_cls.__name__} does not accept the keys {sorted(extra)}")
    return obj


def make_registry(registry_name: str, base_class: type | None = None):
    """Create (or fetch) the registry called ``registry_name``."""
    table = _REGISTRIES.setdefault(registry_name, {})

    def register(name: str, cfg_cls: type | None = None) -> Callable[[type], type]:
        def deco(cls: type) -> type:
            if name in table and table[name][0] is not cls:
                raise ValueError(f"{registry_name} registry already has an entry named {name!r}")
            if base_class is not None and not issubclass(cls, base_class):
                raise TypeError(f"{cls.__name__} must derive from {base_class.__name__}")
            table[name] = (cls, cfg_cls)
            return cls

        return deco

    def build(cfg: Any, cast_to: type | None = None, **kwargs: Any) -> Any:
        if cfg is None:
            return None
        user = _to_plain_dict(cfg)
        name = user.get("_name")
        if name is None:
            raise ValueError(f"{registry_name} config has no '_name': {user}")
        if name not in table:
            raise ValueError(f"unknown {registry_name} {name!r}; registered: {sorted(table)}")
        cls, cfg_cls = table[name]
        full = instantiate_config(cast_to or cfg_cls, user)
        return cls(full, **kwargs)

    return table, register, build


def build(registry_name: str, cfg: Any, **kwargs: Any) -> Any:
    """Module-level convenience: build from the registry called ``registry_name``."""
    if registry_name not in _REGISTRIES:
        raise ValueError(f"no registry named {registry_name!r}")
    return make_registry(registry_name)[2](cfg, **kwargs)
