"""One registry from the architecture's name (config.json `architectures[0]`)
to its typed configuration, as `arch_name` + the `match` of the reference do
(src/arch/mod.rs:33-37, src/main.rs:33-45)."""
from __future__ import annotations

import json
import os
from typing import Any, Callable, Dict

from .llama import ConfigError, LlamaConfig

# name -> function(config dict) -> typed config with .model_spec() and .to_dict()
_ARCHITECTURES: Dict[str, Callable[[Dict[str, Any]], Any]] = {}


def register_architecture(name: str, from_dict: Callable[[Dict[str, Any]], Any]) -> None:
    _ARCHITECTURES[name] = from_dict


def architectures():
    return sorted(_ARCHITECTURES)


def config_from_dict(d: Dict[str, Any]):
    archs = d.get("architectures")
    if not archs:
        raise ConfigError("missing config key: architectures")
    name = archs[0]
    if name not in _ARCHITECTURES:
        raise ConfigError(f"unsupported architecture: {name} (known: {', '.join(architectures())})")
    return _ARCHITECTURES[name](d)


def load_config(path: str):
    """`path` is a model folder or its config.json."""
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    try:
        with open(path) as f:
            d = json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"no config.json at {path}") from None
    return config_from_dict(d)


register_architecture("LlamaForCausalLM", LlamaConfig.from_dict)
