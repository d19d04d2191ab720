"""Typed model configurations and the one registry from architecture name to model.

An architecture is three things: a typed configuration read from its own config.json
keys, a function that turns the configuration into a plan of layers (data: parts chosen
layer by layer and the order they run in), and a table from each part's parameter names
to the tensor names of the model folder.  Counterpart of the reference's flat
`BnConfig` (include/model_config.h:15-53) and its ordered architecture table
(src/model_arch.c:862-987); unlike that table there is no catch-all row: an unknown
architecture is an error.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Callable, Dict, Optional


class ConfigError(ValueError):
    """A config.json that the architecture cannot accept."""


@dataclass(frozen=True)
class Architecture:
    name: str
    config_cls: type                       # has from_dict(dict) and to_dict()
    build_plan: Callable                   # config -> engine.plan.ModelPlan
    aliases: tuple = ()


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(arch: Architecture, *, replace: bool = False) -> Architecture:
    for key in (arch.name,) + tuple(arch.aliases):
        if key in _ARCHITECTURES and not replace:
            raise ValueError(f"architecture {key!r} is already registered")
        _ARCHITECTURES[key] = arch
    return arch


def architecture_names():
    return sorted(_ARCHITECTURES)


def architecture_for(raw: dict) -> Architecture:
    """Choose by `model_type`, then by the entries of `architectures`."""
    keys = []
    if raw.get("model_type"):
        keys.append(str(raw["model_type"]))
    keys += [str(a) for a in raw.get("architectures") or []]
    for key in keys:
        if key in _ARCHITECTURES:
            return _ARCHITECTURES[key]
    raise ConfigError(
        f"no registered architecture for model_type/architectures {keys or '(none given)'}; "
        f"known: {architecture_names()}")


def read_config_json(folder: str) -> dict:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{folder}: no config.json")
    with open(path) as f:
        raw = json.load(f)
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: not a JSON object")
    return raw


def load_config(folder: str):
    """(architecture, typed config) of a model folder."""
    raw = read_config_json(folder)
    arch = architecture_for(raw)
    return arch, arch.config_cls.from_dict(raw)


def _positive_int(raw: dict, key: str, default: Optional[int] = None) -> int:
    v = raw.get(key, default)
    if v is None:
        raise ConfigError(f"config.json: missing key {key!r}")
    if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
        raise ConfigError(f"config.json: {key} must be a positive integer, got {v!r}")
    return v
