"""One registry from an architecture's name (``architectures[0]`` of config.json) to its typed
configuration and the function that turns the configuration into a ModelSpec.  The reference
keeps the same table in its converter (tools/convert.py:29, :56-58)."""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable, Dict, Mapping, Optional

from .config.llama import ConfigError, LlamaConfig
from .models.llama import TINY_LLAMA, llama_spec
from .parts.base import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    config_from_dict: Callable[[Mapping[str, Any]], Any]
    spec_from_config: Callable[[Any], ModelSpec]
    tiny_config: Optional[Mapping[str, Any]] = None     # a small config.json of this architecture for simulations and smoke runs


ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_from_dict, spec_from_config, tiny_config=None) -> None:
    if name in ARCHITECTURES:
        raise ValueError(f"architecture '{name}' is already registered")
    ARCHITECTURES[name] = Architecture(name, config_from_dict, spec_from_config, tiny_config)


def architecture_of(config: Mapping[str, Any]) -> Architecture:
    archs = config.get("architectures")
    if not isinstance(archs, (list, tuple)) or not archs:
        raise ConfigError("config.json lacks 'architectures': [name]")
    arch = ARCHITECTURES.get(archs[0])
    if arch is None:
        raise ConfigError(f"unsupported architecture {archs[0]}; registered: {sorted(ARCHITECTURES)}")
    return arch


def read_config(folder: str | Path) -> Dict[str, Any]:
    path = Path(folder) / "config.json"
    if not path.exists():
        raise ConfigError(f"cannot open {path}")
    return json.loads(path.read_text())


register_architecture("LlamaForCausalLM", LlamaConfig.from_dict, llama_spec, TINY_LLAMA)
