"""One registry from an architecture's name (``config.json["architectures"][0]``) to
everything the engine needs to run it.

The reference picks its model class with if/elif on flags of ``ModelParams``
(reference: torchllms/models/networks.py:779-788) and sniffs the architecture name
while converting checkpoints (torchllms/models/checkpoint_converter.py:323-327); here the
name in config.json is the only key.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable, Dict, List

from .llama import ConfigError, LlamaConfig, llama_model_spec
from .spec import ModelSpec


@dataclass(frozen=True)
class ArchSpec:
    """What an architecture registers.

    ``config_from_dict``  config.json contents -> typed configuration
    ``model_spec``        typed configuration  -> ``ModelSpec`` (parts, sizes, order)
    ``weight_rules``      typed configuration  -> list of ``weights.names.NameRule`` that map
                          checkpoint tensor names to the parts' own names
    """

    name: str
    config_from_dict: Callable[[Dict[str, Any]], Any]
    model_spec: Callable[[Any], ModelSpec]
    weight_rules: Callable[[Any], List[Any]]


ARCHITECTURES: Dict[str, ArchSpec] = {}


def register_architecture(arch: ArchSpec) -> ArchSpec:
    ARCHITECTURES[arch.name] = arch
    return arch


def get_architecture(name: str) -> ArchSpec:
    try:
        return ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(
            f"architecture {name!r} is not registered; registered: {sorted(ARCHITECTURES)}"
        ) from None


def architecture_name(config_dict: Dict[str, Any]) -> str:
    archs = config_dict.get("architectures")
    if not archs:
        raise ConfigError('config.json has no "architectures" entry')
    return archs[0]


def load_config(folder) -> tuple:
    """Read ``folder/config.json``; return ``(ArchSpec, typed configuration)``."""
    path = Path(folder) / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"{path} not found")
    with open(path) as f:
        d = json.load(f)
    arch = get_architecture(architecture_name(d))
    return arch, arch.config_from_dict(d)


def _llama_rules(cfg: LlamaConfig):
    from ..weights.names import llama_name_rules

    return llama_name_rules(cfg)


register_architecture(
    ArchSpec(
        name="LlamaForCausalLM",
        config_from_dict=LlamaConfig.from_dict,
        model_spec=llama_model_spec,
        weight_rules=_llama_rules,
    )
)
