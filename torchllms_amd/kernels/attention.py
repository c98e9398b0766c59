"""Chooses the attention kernel for a step.

float32 always takes the plain kernel, whose result for a token depends only on that token's
position and the cache contents.  bfloat16 takes the MFMA kernels where they support the sizes and
the plain kernel otherwise.
"""

from __future__ import annotations

import torch

from . import ops


def paged_attention(
    qkv: torch.Tensor,
    n_q_heads: int,
    n_kv_heads: int,
    head_dim: int,
    k_pages: torch.Tensor,
    v_pages: torch.Tensor,
    ctx,
    group: int,
    window: int,
    scale: float,
) -> torch.Tensor:
    """Attention of this step's queries (first Hq * dh columns of ``qkv``) over their requests'
    cached keys and values; returns [n_tokens, Hq * dh]."""
    return ops.attention_generic(
        qkv, n_q_heads, n_kv_heads, head_dim, k_pages, v_pages, ctx.token_seq, ctx.positions,
        ctx.block_tables[group], window, scale,
    )
