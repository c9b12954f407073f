"""The one registry from an architecture's name to its model.

``config.json`` names the architecture in ``architectures[0]``; the registry
maps that name to a configuration class (``from_dict(raw) -> config``) and a
builder (``config -> ModelSpec``).  The reference gates on the name with an
``if`` (/root/reference/crates/nnis-model/src/safetensors_loader.rs:137-145);
the error text keeps its style.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, List

from ..errors import InvalidInput, Unsupported


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: Any  # has from_dict(raw) -> typed configuration
    build_spec: Callable[[Any], Any]  # typed configuration -> ModelSpec


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_class: Any, build_spec: Callable[[Any], Any], replace: bool = False) -> None:
    if name in _ARCHITECTURES and not replace:
        raise InvalidInput(f"architecture {name!r} is already registered")
    _ARCHITECTURES[name] = Architecture(name, config_class, build_spec)


def registered_architectures() -> List[str]:
    return sorted(_ARCHITECTURES)


def lookup_architecture(raw_config: Dict[str, Any]) -> Architecture:
    names = raw_config.get("architectures")
    if not isinstance(names, list) or len(names) != 1 or not isinstance(names[0], str):
        raise InvalidInput(f"config.json architectures must be a list with one name; got {names!r}")
    entry = _ARCHITECTURES.get(names[0])
    if entry is None:
        raise Unsupported(
            f"unsupported architecture {names!r} / model_type {raw_config.get('model_type')!r}; "
            f"registered: {', '.join(registered_architectures()) or 'none'}"
        )
    return entry


def spec_from_config(raw_config: Dict[str, Any]):
    """config.json contents -> (typed configuration, ModelSpec)."""
    entry = lookup_architecture(raw_config)
    cfg = entry.config_class.from_dict(raw_config)
    return cfg, entry.build_spec(cfg)
