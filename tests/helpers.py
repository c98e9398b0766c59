"""Shared by the tests: tiny configurations, model folders in temporary places, readers for the
plain implementation."""

from __future__ import annotations

import json
from pathlib import Path
from typing import Dict, List

import torch

# Three tiny configurations of the architecture that differ in every size and option.
TINY_A = {
    "architectures": ["LlamaForCausalLM"],
    "hidden_size": 64,
    "num_hidden_layers": 2,
    "num_attention_heads": 4,
    "num_key_value_heads": 2,
    "intermediate_size": 192,
    "vocab_size": 256,
    "max_position_embeddings": 128,
    "rms_norm_eps": 1e-5,
    "rope_theta": 10000.0,
    "rope_scaling": None,
    "tie_word_embeddings": True,
}
TINY_B = {
    "architectures": ["LlamaForCausalLM"],
    "hidden_size": 256,
    "num_hidden_layers": 3,
    "num_attention_heads": 8,
    "num_key_value_heads": 1,
    "head_dim": 32,
    "intermediate_size": 688,
    "vocab_size": 512,
    "max_position_embeddings": 256,
    "rms_norm_eps": 1e-6,
    "rope_theta": 500000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 8.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 4.0,
        "original_max_position_embeddings": 64,
    },
    "tie_word_embeddings": False,
}
# width, vocabulary and feed-forward that are no power of two, head_dim given apart from
# hidden/heads, three kv groups, biases on q/k/v
TINY_C = {
    "architectures": ["LlamaForCausalLM"],
    "hidden_size": 96,
    "num_hidden_layers": 1,
    "num_attention_heads": 6,
    "num_key_value_heads": 3,
    "head_dim": 48,
    "intermediate_size": 208,
    "vocab_size": 301,
    "max_position_embeddings": 512,
    "rms_norm_eps": 3e-4,
    "rope_theta": 1000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 4.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 2.0,
        "original_max_position_embeddings": 32,
    },
    "tie_word_embeddings": False,
    "attention_bias": True,
}
TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C}
PAGE_SIZE = {"A": 8, "B": 16, "C": 4}


def make_folder(tmp_path, cfg_dict: dict, seed: int = 0, dtype=torch.bfloat16, norm_jitter: float = 0.1,
                sharpen: bool = False) -> Path:
    """A model folder with random weights, made by the package's random-weights mode.

    ``sharpen``: N(0, 0.02) weights give nearly uniform attention, in which one wrong or missing
    key hardly shows.  Scaling the q and k projections so that scores have a spread of about 4
    makes every query attend to a few keys, near and far, and a fault in any of them shows."""
    from safetensors.torch import save_file

    from torchllms_amd.config import LlamaConfig
    from torchllms_amd.weights import write_model_folder

    cfg = LlamaConfig.from_dict(cfg_dict)
    folder = write_model_folder(tmp_path, cfg, seed=seed, dtype=dtype, norm_jitter=norm_jitter)
    if sharpen:
        _, tensors = read_folder(folder)
        factor = 100.0 / cfg.hidden_size ** 0.5
        for name in list(tensors):
            if name.endswith("q_proj.weight") or name.endswith("k_proj.weight"):
                tensors[name] = (tensors[name].float() * factor).to(dtype)
        save_file(tensors, str(folder / "model.safetensors"), metadata={"format": "pt"})
    return folder


def read_folder(folder) -> (dict, Dict[str, torch.Tensor]):
    """config.json as a dict and the tensors by their checkpoint names, read with safetensors
    directly (not through the package's loader)."""
    from safetensors import safe_open

    folder = Path(folder)
    with open(folder / "config.json") as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(str(folder / "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name)
    return cfg, tensors


def random_tokens(n: int, vocab: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
