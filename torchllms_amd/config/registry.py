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
from typing import Any, Callable, Dict, List, Optional, Sequence

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
    #: typed configuration -> the token ids that end a generation when the caller names none
    #: (the checkpoint's end-of-sequence ids); None: the architecture has none to offer
    stop_token_ids: Optional[Callable[[Any], Sequence[int]]] = None
    #: the class of the typed configuration, so that a configuration alone (no folder, no
    #: config.json) finds its architecture: ``architecture_of``
    config_type: Optional[type] = None

    #: typed configuration -> the contents of a config.json that ``config_from_dict`` reads back
    #: (None: the configuration's own ``to_dict()``, or its fields if it is a dataclass)
    config_to_dict: Optional[Callable[[Any], Dict[str, Any]]] = None

    def config_json(self, config) -> Dict[str, Any]:
        """What a model folder's config.json holds for this configuration; it names this architecture."""
        if self.config_to_dict is not None:
            d = dict(self.config_to_dict(config))
        elif hasattr(config, "to_dict"):
            d = dict(config.to_dict())
        else:
            import dataclasses

            d = dataclasses.asdict(config)
        if not d.get("architectures"):
            d["architectures"] = [self.name]
        return d

    def default_stop_token_ids(self, config) -> List[int]:
        return [] if self.stop_token_ids is None else [int(t) for t in self.stop_token_ids(config)]


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


def architecture_of(config) -> ArchSpec:
    """The registered architecture of a typed configuration: the one whose ``config_type`` is the
    configuration's class.  Where several share a class (or none names one) the configuration has
    to say which it is, by an ``architectures`` attribute as config.json has."""
    matches = [a for a in ARCHITECTURES.values() if a.config_type is not None and type(config) is a.config_type]
    if len(matches) == 1:
        return matches[0]
    names = getattr(config, "architectures", None)
    if names:
        return get_architecture(names[0])
    raise ConfigError(
        f"no registered architecture names {type(config).__name__} as its config_type, and the configuration "
        f"has no 'architectures' entry; registered: {sorted(ARCHITECTURES)}"
    )


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


def _llama_stop_ids(cfg: LlamaConfig):
    """config.json's ``eos_token_id``: one id or a list (reference: llm.py:188-200 falls back to the
    tokenizer's eos id, which is this id for the checkpoints it loads)."""
    eos = cfg.eos_token_id
    return [] if eos is None else (list(eos) if isinstance(eos, (list, tuple)) else [eos])


register_architecture(
    ArchSpec(
        name="LlamaForCausalLM",
        config_from_dict=LlamaConfig.from_dict,
        model_spec=llama_model_spec,
        weight_rules=_llama_rules,
        stop_token_ids=_llama_stop_ids,
        config_type=LlamaConfig,
    )
)
