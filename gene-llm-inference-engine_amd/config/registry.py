"""One registry from an architecture's name to its configuration class.

config.json names its architecture in `architectures[0]` (for instance "LlamaForCausalLM");
files without that key are matched by `model_type`.  The reference has no registry: one class
serves its two model types through a flag (src/loader/hf_checkpoint.cpp:96-111).  Here every
architecture registers a configuration class with `from_dict(dict)` and `model_spec()`, from its
own module; this one names none of them.
"""
from __future__ import annotations

import json
from pathlib import Path
from typing import Dict

from .errors import ConfigError

_BY_ARCHITECTURE: Dict[str, type] = {}
_BY_MODEL_TYPE: Dict[str, str] = {}


def register_architecture(name: str, config_class: type, model_type: str | None = None) -> None:
    """`config_class.from_dict(config_json_dict)` must give an object with `model_spec()`."""
    if name in _BY_ARCHITECTURE and _BY_ARCHITECTURE[name] is not config_class:
        raise ValueError(f"architecture '{name}' is already registered")
    _BY_ARCHITECTURE[name] = config_class
    if model_type is not None:
        _BY_MODEL_TYPE[model_type] = name


def registered_architectures():
    return sorted(_BY_ARCHITECTURE)


def config_class_for(cfg: dict) -> type:
    if not isinstance(cfg, dict):
        raise ConfigError("config.json is not a JSON object")
    archs = cfg.get("architectures")
    if isinstance(archs, list) and archs:
        name = archs[0]
    else:
        name = _BY_MODEL_TYPE.get(cfg.get("model_type"))
    if name not in _BY_ARCHITECTURE:
        shown = repr(name) if name is not None else f"(model_type {cfg.get('model_type')!r}, no 'architectures')"
        raise ConfigError(f"unknown architecture {shown}; registered: {', '.join(registered_architectures())}")
    return _BY_ARCHITECTURE[name]


def parse_config(cfg: dict):
    """The typed configuration of whichever architecture config.json names."""
    return config_class_for(cfg).from_dict(cfg)


def read_config(folder):
    path = Path(folder) / "config.json"
    if not path.exists():
        raise ConfigError(f"no config.json in {folder}")
    try:
        cfg = json.loads(path.read_text())
    except json.JSONDecodeError as e:
        raise ConfigError(f"config.json: {e}") from None
    return parse_config(cfg)

