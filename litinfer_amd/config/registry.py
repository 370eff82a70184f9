"""One registry from the architecture's name to its model definition.

An architecture is a typed configuration class with `from_dict` and a function
from that configuration to a `ModelSpec`; beside them it may name other names
under which checkpoints store its tensors (`weight_aliases`: stored name ->
the model's name) and an entry class of its own for `models.load` (the generic
one otherwise).  The name comes from config.json (`architectures[0]`, else
`model_type`).  This is the only table from names to models: loading, the
command line, replay and the benchmark all look here.
"""
from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from dataclasses import field
from typing import Any, Callable, Dict, Mapping, Optional, Tuple

from .spec import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    config_from_dict: Callable[[Dict[str, Any]], Any]
    model_spec: Callable[[Any], ModelSpec]
    weight_aliases: Mapping[str, str] = field(default_factory=dict)
    entry: Optional[type] = None


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_from_dict, model_spec, aliases=(), weight_aliases=None,
                          entry=None) -> None:
    """`aliases`: further names of the architecture.  `weight_aliases`: stored tensor
    name -> the name the model's parts use.  `entry`: the class that `models.load`
    builds for a model folder of this architecture (default: the generic one)."""
    arch = Architecture(name, config_from_dict, model_spec, dict(weight_aliases or {}), entry)
    for n in (name, *aliases):
        _ARCHITECTURES[n] = arch


def registered_architectures():
    return sorted(_ARCHITECTURES)


def architecture_name(cfg: Dict[str, Any]) -> str:
    archs = cfg.get("architectures")
    if isinstance(archs, list) and archs:
        return str(archs[0])
    if cfg.get("model_type"):
        return str(cfg["model_type"])
    raise ValueError("config.json names no architecture (keys 'architectures', 'model_type')")


def lookup(name: str) -> Architecture:
    if name not in _ARCHITECTURES:
        raise KeyError(f"unknown architecture '{name}'; registered: "
                       f"{', '.join(registered_architectures())}")
    return _ARCHITECTURES[name]


def read_config_json(model_dir) -> Dict[str, Any]:
    path = Path(model_dir) / "config.json"
    if not path.exists():
        raise FileNotFoundError(f"Config file not found: {path}")
    with open(path, "r", encoding="utf-8") as f:
        return json.load(f)


def load_config(model_dir) -> Tuple[Architecture, Any, ModelSpec]:
    """(architecture, typed configuration, model spec) of a model folder."""
    raw = read_config_json(model_dir)
    arch = lookup(architecture_name(raw))
    cfg = arch.config_from_dict(raw)
    spec = arch.model_spec(cfg)
    spec.validate()
    return arch, cfg, spec
