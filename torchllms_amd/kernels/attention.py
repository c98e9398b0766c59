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
    n = qkv.shape[0]
    n_dec = ctx.host.n_decode
    fast_decode = n_dec > 0 and ops.decode_attention_supported(qkv.dtype, n_q_heads, n_kv_heads, head_dim)
    if not fast_decode:
        return ops.attention_generic(
            qkv, n_q_heads, n_kv_heads, head_dim, k_pages, v_pages, ctx.token_seq, ctx.positions,
            ctx.block_tables[group], window, scale,
        )
    out = torch.empty((n, n_q_heads * head_dim), dtype=qkv.dtype, device=qkv.device)
    # rows with a single new token come first in the batch: they take the split-KV decode kernel
    if ctx.decode_longest is not None:
        longest = ctx.decode_longest
    else:
        longest = int(ctx.host.positions[:n_dec].max()) + 1
    if window > 0:
        longest = min(longest, window + 15)
    ops.attention_decode(
        qkv[:n_dec], n_q_heads, n_kv_heads, head_dim, k_pages, v_pages, ctx.token_seq[:n_dec], ctx.positions[:n_dec],
        ctx.block_tables[group], window, scale, longest, out=out[:n_dec],
    )
    if n_dec < n:
        ops.attention_generic(
            qkv[n_dec:], n_q_heads, n_kv_heads, head_dim, k_pages, v_pages, ctx.token_seq[n_dec:], ctx.positions[n_dec:],
            ctx.block_tables[group], window, scale, out=out[n_dec:],
        )
    return out
