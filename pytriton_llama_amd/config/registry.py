"""One registry from an architecture's name to its configuration class and
model builder. The reference dispatches on ``model_type`` with if/elif chains
in three places (lite_llama/executor/model_executor.py:31-36,141-153,170-179)
and never consults ``architectures``; here ``architectures[0]`` of config.json
is the key everywhere.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict

from .model_config import ConfigError, read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: Any                       # has from_dict(dict)
    build: Callable[[Any], Any]             # typed config -> model (no weights yet)


MODEL_REGISTRY: Dict[str, Architecture] = {}
# config.json files without an "architectures" entry are recognised by their model_type
MODEL_TYPE_ALIASES: Dict[str, str] = {}


def register_model(name: str, config_class, build, model_type: str = None) -> None:
    MODEL_REGISTRY[name] = Architecture(name, config_class, build)
    if model_type:
        MODEL_TYPE_ALIASES[model_type] = name


def architecture_of(config_dict: Dict[str, Any]) -> Architecture:
    archs = config_dict.get("architectures")
    if not archs and config_dict.get("model_type") in MODEL_TYPE_ALIASES:
        archs = [MODEL_TYPE_ALIASES[config_dict["model_type"]]]
    if not archs:
        raise ConfigError("config.json has no 'architectures' entry; "
                          f"supported: {sorted(MODEL_REGISTRY)}")
    name = archs[0]
    if name not in MODEL_REGISTRY:
        raise ConfigError(f"architecture {name!r} is not supported; "
                          f"supported: {sorted(MODEL_REGISTRY)}")
    return MODEL_REGISTRY[name]


def config_from_dict(config_dict: Dict[str, Any]):
    return architecture_of(config_dict).config_class.from_dict(config_dict)


def config_from_folder(folder: str):
    return config_from_dict(read_config_json(folder))


def build_model(config_dict_or_typed):
    """A model object (parts wired, no weights loaded) for a config dict."""
    if isinstance(config_dict_or_typed, dict):
        arch = architecture_of(config_dict_or_typed)
        cfg = arch.config_class.from_dict(config_dict_or_typed)
    else:
        cfg = config_dict_or_typed
        arch = MODEL_REGISTRY[cfg.architectures[0]]
    return arch.build(cfg)
