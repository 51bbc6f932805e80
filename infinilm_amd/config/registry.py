"""One registry from an architecture's name to (typed configuration, model description).

Role of csrc/models/models_registry.{hpp,cpp} and model_factory.cpp:6-26 in the reference: a name
from config.json selects how the configuration is completed and which model is built.  Lookup
goes by `architectures[0]` first, then by `model_type`.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict, Iterable

from .errors import ConfigError
from .spec import ModelSpec


@dataclass
class Architecture:
    name: str
    config_from_dict: Callable[[Dict[str, Any]], Any]
    build_spec: Callable[[Any], ModelSpec]


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(names: Iterable[str], config_from_dict, build_spec) -> None:
    """`names`: every `architectures` entry and `model_type` value that selects this model."""
    names = list(names)
    arch = Architecture(names[0], config_from_dict, build_spec)
    for n in names:
        _ARCHITECTURES[n] = arch


def registered_architectures():
    return sorted(_ARCHITECTURES)


def resolve_architecture(raw: Dict[str, Any]) -> Architecture:
    tried = []
    archs = raw.get("architectures") or []
    if isinstance(archs, str):
        archs = [archs]
    for n in list(archs) + [raw.get("model_type")]:
        if n is None:
            continue
        tried.append(str(n))
        if n in _ARCHITECTURES:
            return _ARCHITECTURES[n]
    raise ConfigError("Unsupported model_type: none of " + repr(tried) + " is registered; known: "
                      + ", ".join(registered_architectures()))


def read_config_json(model_dir: str) -> Dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{path} not found")
    with open(path) as fh:
        raw = json.load(fh)
    if not isinstance(raw, dict):
        raise ConfigError(f"{path} does not hold a JSON object")
    gen = os.path.join(model_dir, "generation_config.json")
    if os.path.isfile(gen):  # eos ids: generation_config.json first (python/infinilm/infer_engine.py:231-252)
        try:
            with open(gen) as fh:
                g = json.load(fh)
            if "eos_token_id" in g:
                raw = dict(raw, eos_token_id=g["eos_token_id"])
        except (OSError, ValueError):
            pass
    return raw


def load_model_config(model_dir_or_dict):
    """(architecture, typed configuration) from a model folder or an already parsed config.json."""
    from .. import models  # noqa: F401  (registers the built-in architecture)

    raw = model_dir_or_dict if isinstance(model_dir_or_dict, dict) else read_config_json(model_dir_or_dict)
    arch = resolve_architecture(raw)
    return arch, arch.config_from_dict(raw)
