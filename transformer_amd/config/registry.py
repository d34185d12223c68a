"""One registry from an architecture's name to what builds its model.

An entry supplies three things: how to read the typed configuration, how to
spell the model out as blocks and a schedule, and where each parameter of
those blocks is found in a weight file. The cache, the step function, the
generation loop, trace replay and the bench never look at the name.

The reference has no such table: its crates are the registry
(Cargo.toml:8-18) and ``general.architecture`` only switches
one bias (models/llama/common/src/storage.rs:31,45).
"""
from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Callable, Dict

from .spec import ConfigError


class UnknownArchitecture(ConfigError):
    pass


@dataclass(frozen=True)
class Architecture:
    name: str
    config_from_dict: Callable      # config.json dict -> typed config
    config_from_gguf: Callable      # (metadata dict, vocab rows) -> typed config, or None
    model_spec: Callable            # typed config -> ModelSpec
    weight_sources: Callable        # (typed config, ModelSpec, file format) -> {param: Source}


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(arch: Architecture, *aliases: str) -> None:
    for n in (arch.name, *aliases):
        _ARCHITECTURES[n] = arch


def known_architectures():
    return sorted(_ARCHITECTURES)


def get_architecture(name: str) -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise UnknownArchitecture(
            f"unknown architecture {name!r}; known: {', '.join(known_architectures())}") from None


def architecture_of_config_json(d: dict) -> Architecture:
    """config.json names its model class in ``architectures`` (first entry);
    ``model_type`` is the fallback."""
    names = d.get("architectures")
    if isinstance(names, (list, tuple)) and names:
        return get_architecture(names[0])
    if "model_type" in d:
        return get_architecture(d["model_type"])
    raise ConfigError("config.json has neither 'architectures' nor 'model_type'")


def read_model_folder_config(folder):
    """(architecture entry, typed config) of a folder holding config.json."""
    p = Path(folder) / "config.json"
    try:
        d = json.loads(p.read_text())
    except FileNotFoundError:
        raise ConfigError(f"no config.json in {folder}") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{p}: not valid JSON ({e})") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{p}: top level must be an object")
    arch = architecture_of_config_json(d)
    return arch, arch.config_from_dict(d)
