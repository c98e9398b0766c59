"""Tensor-name rules: checkpoint names -> the parts' own names, with re-layouts.

Two spellings of the Llama 3 decoder are accepted:

* the checkpoint's own (``model.layers.3.self_attn.q_proj.weight`` ...), whose q/k rows are
  laid out for half-split rotary pairs ``(i, i + head_dim/2)``;
* the reference's internal one (``layers.3.attention.wq.weight`` ...), whose q/k rows are
  already laid out for interleaved pairs ``(2i, 2i+1)``.

The name table and the row permutation restate
reference: torchllms/models/checkpoint_converter.py:96-108 (permute), 124-141 (names),
199-229 (inverse).  The engine rotates interleaved pairs (reference:
torchllms/models/networks.py:332-352), so checkpoint-spelled q/k tensors are permuted on load.
"""

from __future__ import annotations

import re
from dataclasses import dataclass
from typing import Callable, List, Optional, Tuple

import torch


def half_split_to_interleaved(w: torch.Tensor, n_heads: int, head_dim: int) -> torch.Tensor:
    """Reorder rows of a q/k projection (or entries of its bias) so that the element that sat
    at offset ``i`` / ``i + head_dim/2`` of each head sits at ``2i`` / ``2i + 1``."""
    if w.shape[0] != n_heads * head_dim:
        raise ValueError(f"expected leading size {n_heads * head_dim}, got {tuple(w.shape)}")
    rest = w.shape[1:]
    return w.reshape(n_heads, 2, head_dim // 2, *rest).transpose(1, 2).reshape(n_heads * head_dim, *rest)


def interleaved_to_half_split(w: torch.Tensor, n_heads: int, head_dim: int) -> torch.Tensor:
    """Inverse of :func:`half_split_to_interleaved`."""
    if w.shape[0] != n_heads * head_dim:
        raise ValueError(f"expected leading size {n_heads * head_dim}, got {tuple(w.shape)}")
    rest = w.shape[1:]
    return w.reshape(n_heads, head_dim // 2, 2, *rest).transpose(1, 2).reshape(n_heads * head_dim, *rest)


@dataclass(frozen=True)
class NameRule:
    """``external`` and ``internal`` are patterns in which ``{}`` stands for a layer index.

    ``load`` re-lays a tensor out on the way in, ``save`` on the way out (both None: as is).
    ``internal=None`` means: a tensor of this name is known and dropped.
    """

    external: str
    internal: Optional[str]
    load: Optional[Callable[[torch.Tensor], torch.Tensor]] = None
    save: Optional[Callable[[torch.Tensor], torch.Tensor]] = None

    def _regex(self, pattern: str) -> "re.Pattern":
        return re.compile("^" + re.escape(pattern).replace(re.escape("{}"), r"(\d+)") + "$")

    def match_external(self, name: str) -> Optional[Tuple[Optional[str]]]:
        m = self._regex(self.external).match(name)
        if m is None:
            return None
        if self.internal is None:
            return (None,)
        return (self.internal.format(*m.groups()),)

    def match_internal(self, name: str) -> Optional[str]:
        if self.internal is None:
            return None
        m = self._regex(self.internal).match(name)
        if m is None:
            return None
        return self.external.format(*m.groups())


def llama_name_rules(cfg) -> List[NameRule]:
    """Rules for both spellings.  The checkpoint spelling comes first, so it is the one
    used when a model folder is written."""
    hq, hkv, dh = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim

    def perm(h):
        return (
            lambda w: half_split_to_interleaved(w, h, dh),
            lambda w: interleaved_to_half_split(w, h, dh),
        )

    q_in, q_out = perm(hq)
    k_in, k_out = perm(hkv)
    L = "model.layers.{}."
    I = "layers.{}."
    rules = [
        NameRule("model.embed_tokens.weight", "embed.weight"),
        NameRule(L + "self_attn.q_proj.weight", I + "mixer.wq.weight", q_in, q_out),
        NameRule(L + "self_attn.q_proj.bias", I + "mixer.wq.bias", q_in, q_out),
        NameRule(L + "self_attn.k_proj.weight", I + "mixer.wk.weight", k_in, k_out),
        NameRule(L + "self_attn.k_proj.bias", I + "mixer.wk.bias", k_in, k_out),
        NameRule(L + "self_attn.v_proj.weight", I + "mixer.wv.weight"),
        NameRule(L + "self_attn.v_proj.bias", I + "mixer.wv.bias"),
        NameRule(L + "self_attn.o_proj.weight", I + "mixer.wo.weight"),
        NameRule(L + "self_attn.rotary_emb.inv_freq", None),
        NameRule(L + "mlp.gate_proj.weight", I + "ffn.w1.weight"),
        NameRule(L + "mlp.up_proj.weight", I + "ffn.w3.weight"),
        NameRule(L + "mlp.down_proj.weight", I + "ffn.w2.weight"),
        NameRule(L + "input_layernorm.weight", I + "mixer_norm.weight"),
        NameRule(L + "post_attention_layernorm.weight", I + "ffn_norm.weight"),
        NameRule("model.norm.weight", "final_norm.weight"),
        NameRule("lm_head.weight", "head.weight"),
        # the reference's internal spelling, taken as is
        NameRule("tok_embeddings.weight", "embed.weight"),
        NameRule(I + "attention.wq.weight", I + "mixer.wq.weight"),
        NameRule(I + "attention.wq.bias", I + "mixer.wq.bias"),
        NameRule(I + "attention.wk.weight", I + "mixer.wk.weight"),
        NameRule(I + "attention.wk.bias", I + "mixer.wk.bias"),
        NameRule(I + "attention.wv.weight", I + "mixer.wv.weight"),
        NameRule(I + "attention.wv.bias", I + "mixer.wv.bias"),
        NameRule(I + "attention.wo.weight", I + "mixer.wo.weight"),
        NameRule(I + "feed_forward.w1.weight", I + "ffn.w1.weight"),
        NameRule(I + "feed_forward.w3.weight", I + "ffn.w3.weight"),
        NameRule(I + "feed_forward.w2.weight", I + "ffn.w2.weight"),
        NameRule(I + "attention_norm.weight", I + "mixer_norm.weight"),
        NameRule(I + "ffn_norm.weight", I + "ffn_norm.weight"),
        NameRule("norm.weight", "final_norm.weight"),
        NameRule("output.weight", "head.weight"),
    ]
    return rules
