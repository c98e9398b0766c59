"""Typed configuration of the Llama 3 dense decoder, read from ``config.json``.

Key names are those of the checkpoint's own ``config.json``.  The reference maps the same
keys into its ``ModelParams`` (reference: torchllms/models/checkpoint_converter.py:359-397,
torchllms/models/networks.py:110-157); here they are read directly, and
``intermediate_size`` is taken as given instead of being re-derived from
``ffn_dim_multiplier``/``multiple_of`` (networks.py:595-598).
"""

from __future__ import annotations

import json
from dataclasses import dataclass, field, fields
from pathlib import Path
from typing import Any, Dict, List, Optional

from .spec import LayerRun, LayerSpec, ModelSpec, PartSpec, standard_layer

_ROPE_SCALING_KEYS = (
    "factor",
    "low_freq_factor",
    "high_freq_factor",
    "original_max_position_embeddings",
)


class ConfigError(ValueError):
    """A config.json that cannot describe a model this engine runs."""


@dataclass(frozen=True)
class RopeScaling:
    """``rope_scaling`` of config.json.  ``rope_type`` "default" carries no factors."""

    rope_type: str = "default"
    factor: float = 1.0
    low_freq_factor: float = 1.0
    high_freq_factor: float = 1.0
    original_max_position_embeddings: int = 0

    @classmethod
    def from_dict(cls, d: Optional[Dict[str, Any]]) -> "RopeScaling":
        if not d:
            return cls()
        rope_type = d.get("rope_type", d.get("type", "default"))
        if rope_type == "default":
            return cls()
        if rope_type != "llama3":
            # reference: networks.py:278-279 raises on any other type
            raise ConfigError(f"rope_scaling.rope_type={rope_type!r} is not supported (default, llama3)")
        missing = [k for k in _ROPE_SCALING_KEYS if k not in d]
        if missing:
            raise ConfigError(f"rope_scaling of type llama3 lacks {missing}")
        out = cls(
            rope_type="llama3",
            factor=float(d["factor"]),
            low_freq_factor=float(d["low_freq_factor"]),
            high_freq_factor=float(d["high_freq_factor"]),
            original_max_position_embeddings=int(d["original_max_position_embeddings"]),
        )
        if out.high_freq_factor == out.low_freq_factor:
            raise ConfigError("rope_scaling: high_freq_factor must differ from low_freq_factor")
        if out.factor <= 0 or out.original_max_position_embeddings <= 0:
            raise ConfigError("rope_scaling: factor and original_max_position_embeddings must be positive")
        return out

    def to_dict(self) -> Optional[Dict[str, Any]]:
        if self.rope_type == "default":
            return None
        return {
            "rope_type": self.rope_type,
            "factor": self.factor,
            "low_freq_factor": self.low_freq_factor,
            "high_freq_factor": self.high_freq_factor,
            "original_max_position_embeddings": self.original_max_position_embeddings,
        }


@dataclass(frozen=True)
class LlamaConfig:
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    intermediate_size: int
    vocab_size: int
    max_position_embeddings: int
    num_key_value_heads: Optional[int] = None  # None -> num_attention_heads (networks.py:153-154)
    head_dim: Optional[int] = None  # None -> hidden_size // heads (networks.py:150-151)
    rms_norm_eps: float = 1e-5  # networks.py:120
    rope_theta: float = 10000.0  # networks.py:123
    rope_scaling: RopeScaling = field(default_factory=RopeScaling)
    tie_word_embeddings: bool = False  # networks.py:119
    attention_bias: bool = False  # networks.py:122 (attn_proj_bias)
    torch_dtype: str = "bfloat16"
    bos_token_id: Optional[int] = None
    eos_token_id: Any = None
    architectures: tuple = ("LlamaForCausalLM",)

    def __post_init__(self):
        if self.num_key_value_heads is None:
            object.__setattr__(self, "num_key_value_heads", self.num_attention_heads)
        if self.head_dim is None:
            if self.hidden_size % self.num_attention_heads:
                raise ConfigError("hidden_size is not a multiple of num_attention_heads and head_dim is not given")
            object.__setattr__(self, "head_dim", self.hidden_size // self.num_attention_heads)
        self.validate()

    def validate(self) -> None:
        for name in (
            "hidden_size",
            "num_hidden_layers",
            "num_attention_heads",
            "num_key_value_heads",
            "head_dim",
            "intermediate_size",
            "vocab_size",
            "max_position_embeddings",
        ):
            v = getattr(self, name)
            if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
                raise ConfigError(f"{name} must be a positive integer, got {v!r}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads={self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads={self.num_key_value_heads}"
            )
        if self.head_dim % 2:
            raise ConfigError(f"head_dim={self.head_dim} must be even for rotary pairs")
        if not self.rms_norm_eps > 0:
            raise ConfigError(f"rms_norm_eps must be positive, got {self.rms_norm_eps!r}")
        if not self.rope_theta > 0:
            raise ConfigError(f"rope_theta must be positive, got {self.rope_theta!r}")

    # ------------------------------------------------------------------ reading / writing
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LlamaConfig":
        required = [
            "hidden_size",
            "num_hidden_layers",
            "num_attention_heads",
            "intermediate_size",
            "vocab_size",
            "max_position_embeddings",
        ]
        missing = [k for k in required if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks required keys {missing}")
        if d.get("hidden_act", "silu") != "silu":
            raise ConfigError(f"hidden_act={d['hidden_act']!r}: this architecture's feed-forward is SwiGLU (silu)")
        if d.get("mlp_bias", False):
            raise ConfigError("mlp_bias=true: the feed-forward of this architecture has no biases")
        rope_theta = d.get("rope_theta")
        rope_scaling = d.get("rope_scaling")
        # newer config.json files fold both into "rope_parameters"
        rp = d.get("rope_parameters")
        if rp:
            rope_theta = rp.get("rope_theta", rope_theta)
            if rope_scaling is None and rp.get("rope_type", "default") != "default":
                rope_scaling = {k: v for k, v in rp.items() if k != "rope_theta"}
        kw: Dict[str, Any] = dict(
            hidden_size=d["hidden_size"],
            num_hidden_layers=d["num_hidden_layers"],
            num_attention_heads=d["num_attention_heads"],
            intermediate_size=d["intermediate_size"],
            vocab_size=d["vocab_size"],
            max_position_embeddings=d["max_position_embeddings"],
            num_key_value_heads=d.get("num_key_value_heads"),
            head_dim=d.get("head_dim"),
            rope_scaling=RopeScaling.from_dict(rope_scaling),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            attention_bias=bool(d.get("attention_bias", False)),
            torch_dtype=str(d.get("torch_dtype", d.get("dtype", "bfloat16"))),
            bos_token_id=d.get("bos_token_id"),
            eos_token_id=d.get("eos_token_id"),
            architectures=tuple(d.get("architectures", ("LlamaForCausalLM",))),
        )
        # reference: checkpoint_converter.py:386-389 takes these two only when truthy
        if d.get("rms_norm_eps"):
            kw["rms_norm_eps"] = float(d["rms_norm_eps"])
        if rope_theta:
            kw["rope_theta"] = float(rope_theta)
        return cls(**kw)

    @classmethod
    def from_json_file(cls, path) -> "LlamaConfig":
        with open(path) as f:
            return cls.from_dict(json.load(f))

    def to_dict(self) -> Dict[str, Any]:
        d = {f.name: getattr(self, f.name) for f in fields(self)}
        d["rope_scaling"] = self.rope_scaling.to_dict()
        d["architectures"] = list(self.architectures)
        d["hidden_act"] = "silu"
        d["model_type"] = "llama"
        d["mlp_bias"] = False
        return d

    def save(self, folder) -> None:
        folder = Path(folder)
        folder.mkdir(parents=True, exist_ok=True)
        with open(folder / "config.json", "w") as f:
            json.dump(self.to_dict(), f, indent=2)


def llama_model_spec(cfg: LlamaConfig) -> ModelSpec:
    """The Llama 3 decoder as data: ``num_hidden_layers`` pre-norm layers of grouped-query
    attention with rotary positions and a SwiGLU feed-forward, run once each in order
    (reference: networks.py:617-644 block, 790-809 model)."""
    position = PartSpec(
        "rope",
        dict(
            head_dim=cfg.head_dim,
            rotary_dim=cfg.head_dim,
            theta=cfg.rope_theta,
            scaling=cfg.rope_scaling.to_dict(),
            pairing="interleaved",  # networks.py:332-352
        ),
    )
    norm = PartSpec("rmsnorm", dict(size=cfg.hidden_size, eps=cfg.rms_norm_eps))
    mixer = PartSpec(
        "attention",
        dict(
            hidden_size=cfg.hidden_size,
            num_heads=cfg.num_attention_heads,
            num_kv_heads=cfg.num_key_value_heads,
            head_dim=cfg.head_dim,
            qkv_bias=cfg.attention_bias,
            softmax_scale=cfg.head_dim ** -0.5,  # networks.py:842
            window=0,
            position=position,
        ),
    )
    ffn = PartSpec("swiglu", dict(hidden_size=cfg.hidden_size, intermediate_size=cfg.intermediate_size))
    layers: List[LayerSpec] = [
        standard_layer(f"layers.{i}", "pre_norm", mixer=mixer, feed_forward=ffn, mixer_norm=norm, ffn_norm=norm)
        for i in range(cfg.num_hidden_layers)
    ]
    spec = ModelSpec(
        architecture="LlamaForCausalLM",
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        max_positions=cfg.max_position_embeddings,
        embedding=PartSpec("embedding", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size)),
        layers=layers,
        order=[LayerRun(i) for i in range(cfg.num_hidden_layers)],
        final_norm=norm,
        head=PartSpec(
            "lm_head",
            dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, tied=cfg.tie_word_embeddings),
        ),
    )
    spec.validate()
    return spec
