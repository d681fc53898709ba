"""One registry from an architecture's name to its configuration class and model builder.

``config.json["architectures"][0]`` chooses the entry (``model_type`` is the fallback for folders
that omit it). An entry holds the typed configuration's parser and a function that turns a parsed
configuration into a :class:`dli_amd.parts.spec.ModelSpec`: the list of parts that the model is put
together from. Registering a new architecture touches no file of the framework::

    register_architecture("MyModelForCausalLM", MyConfig.from_hf_dict, build_my_spec,
                          model_types=("my_model",))
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable, Mapping

from .errors import ConfigError, UnsupportedModelError


@dataclass(frozen=True)
class Architecture:
    name: str
    parse_config: Callable[[Mapping[str, Any]], Any]
    build_spec: Callable[[Any], Any]
    model_types: tuple[str, ...] = ()


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(
    name: str,
    parse_config: Callable[[Mapping[str, Any]], Any],
    build_spec: Callable[[Any], Any],
    *,
    model_types: tuple[str, ...] = (),
    replace: bool = False,
) -> Architecture:
    """Add an architecture. ``build_spec(config)`` returns the model's ``ModelSpec``."""
    if name in _ARCHITECTURES and not replace:
        raise ConfigError(f"architecture {name!r} is already registered")
    arch = Architecture(name, parse_config, build_spec, tuple(model_types))
    _ARCHITECTURES[name] = arch
    return arch


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def registered_architectures() -> tuple[str, ...]:
    return tuple(sorted(_ARCHITECTURES))


def resolve_architecture(cfg: Mapping[str, Any]) -> Architecture:
    """Pick the registry entry that a ``config.json`` dictionary names."""
    names = cfg.get("architectures") or []
    for name in names:
        if name in _ARCHITECTURES:
            return _ARCHITECTURES[name]
    if not names:
        model_type = cfg.get("model_type")
        for arch in _ARCHITECTURES.values():
            if model_type is not None and model_type in arch.model_types:
                return arch
    raise UnsupportedModelError(
        f"no registered architecture for architectures={list(names)!r}, "
        f"model_type={cfg.get('model_type')!r}; known: {list(registered_architectures())}"
    )


def read_config_json(model_dir: str | Path) -> dict[str, Any]:
    path = Path(model_dir) / "config.json"
    if not path.is_file():
        raise ConfigError(f"{path} does not exist")
    try:
        data = json.loads(path.read_text())
    except json.JSONDecodeError as exc:
        raise ConfigError(f"{path} is not valid JSON: {exc}") from exc
    if not isinstance(data, dict):
        raise ConfigError(f"{path} does not hold a JSON object")
    return data


def load_config(model_dir: str | Path) -> Any:
    """Parse ``config.json`` of ``model_dir`` with the registered architecture's parser."""
    raw = read_config_json(model_dir)
    return resolve_architecture(raw).parse_config(raw)
