"""One registry from an architecture's name to its configuration class.

The reference maps ``"llama" | "LlamaForCausalLM"`` to its block description
(/root/reference/engine/src/architecture.rs:123-135) and silently treats unknown
names as Llama (/root/reference/engine/src/config.rs:102-114); here an unknown
name is an error.
"""
from __future__ import annotations

import json
import os
from typing import Any, Callable, Dict

from .llama import ConfigError, LlamaConfig

_ARCHITECTURES: Dict[str, Any] = {}


def register_architecture(name: str, config_cls) -> None:
    """Register ``config_cls`` under ``name``.

    ``config_cls`` must offer ``from_dict(dict)`` and ``build_spec() -> ModelSpec``
    (and ``to_json()`` if random model folders are to be written for it).
    """
    _ARCHITECTURES[name] = config_cls


def architecture_names():
    return sorted(_ARCHITECTURES)


def config_class_for(name: str):
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(
            f"unknown architecture {name!r}; registered: {', '.join(architecture_names())}") from None


def load_config(model_dir: str):
    """Read ``model_dir/config.json`` and return the typed config its architecture names."""
    path = os.path.join(model_dir, "config.json")
    try:
        with open(path, "r") as f:
            text = f.read()
    except OSError as e:
        raise ConfigError(f"cannot read {path}: {e}") from e
    try:
        d = json.loads(text)
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: malformed JSON: {e}") from e
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    archs = d.get("architectures")
    if isinstance(archs, list) and archs:
        name = archs[0]
    elif d.get("model_type") is not None:
        name = d["model_type"]
    else:
        raise ConfigError(f"{path}: neither 'architectures' nor 'model_type' names the model")
    return config_class_for(str(name)).from_dict(d)


register_architecture("LlamaForCausalLM", LlamaConfig)
register_architecture("llama", LlamaConfig)
