"""Chooses the attention kernel for a step.

float32 always takes the plain kernel, whose result for a token depends only on that token's
position and the cache contents.  bfloat16 takes the MFMA kernels where they support the sizes and
the plain kernel otherwise.
"""

from __future__ import annotations

import torch

from . import ops

#: contexts beyond this many keys give every block of 64 keys a wave of its own in the plain kernel
GENERIC_SPLIT_FROM = 128


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
    # the MFMA prefill kernel takes positive softmax scales only; anything else runs the plain kernel
    fast_prefill = n_dec < n and scale > 0 and ops.prefill_attention_supported(qkv.dtype, n_q_heads, n_kv_heads, head_dim, k_pages.shape[2])
    out = torch.empty((n, n_q_heads * head_dim), dtype=qkv.dtype, device=qkv.device)
    # rows with a single new token come first in the batch
    if n_dec > 0:
        if ctx.decode_longest is not None:
            longest = ctx.decode_longest
        else:
            longest = int(ctx.host.positions[:n_dec].max()) + 1
        if fast_decode:
            # the split-KV MFMA kernel
            if window > 0:
                longest = min(longest, window + 15)
            uneven = ctx.decode_uneven if ctx.decode_uneven is not None else ctx.host.decode_uneven
            ops.attention_decode(
                qkv[:n_dec], n_q_heads, n_kv_heads, head_dim, k_pages, v_pages, ctx.token_seq[:n_dec],
                ctx.positions[:n_dec], ctx.block_tables[group], window, scale, longest, out=out[:n_dec],
                uneven=uneven,
            )
        else:
            # the plain kernel: one wave a (token, head) would walk the whole context alone, so the
            # blocks of 64 keys get waves of their own (the same bits either way)
            if window > 0:
                longest = min(longest, window)
            plain = ops.attention_generic_split if longest > GENERIC_SPLIT_FROM else ops.attention_generic
            extra = dict(longest=longest) if longest > GENERIC_SPLIT_FROM else {}
            plain(
                qkv[:n_dec], n_q_heads, n_kv_heads, head_dim, k_pages, v_pages, ctx.token_seq[:n_dec],
                ctx.positions[:n_dec], ctx.block_tables[group], window, scale, out=out[:n_dec], **extra,
            )
    # rows that bring a portion of a prompt take the tiled MFMA kernel
    if n_dec < n:
        if fast_prefill:
            qpt = ops.prefill_queries_per_tile(n_q_heads, n_kv_heads, head_dim)
            key = ("prefill_tiles", qpt, window, n_kv_heads)
            tiles = ctx.scratch.get(key)
            if tiles is None:
                host = ctx.host
                longest = int(max(host.kv_lens[n_dec : host.n_seqs]))
                if window > 0:
                    longest = min(longest, window + qpt)
                key_groups = ops.prefill_key_groups(ops.prefill_tile_count(host.qo_indptr, n_dec, host.n_seqs, qpt), n_kv_heads, longest)
                rows, q0s = ops.prefill_tiles(host.qo_indptr, n_dec, host.n_seqs, qpt, host.kv_lens, window)
                both = torch.tensor([rows, q0s], dtype=torch.int32).to(qkv.device)
                tiles = (both[0], both[1], key_groups)
                ctx.scratch[key] = tiles
            ops.attention_prefill(
                qkv, n_q_heads, n_kv_heads, head_dim, k_pages, v_pages, ctx.qo_indptr, ctx.kv_lens,
                ctx.block_tables[group], tiles[0], tiles[1], window, scale, out, key_groups=tiles[2],
            )
        else:
            ops.attention_generic(
                qkv[n_dec:], n_q_heads, n_kv_heads, head_dim, k_pages, v_pages, ctx.token_seq[n_dec:],
                ctx.positions[n_dec:], ctx.block_tables[group], window, scale, out=out[n_dec:],
            )
    return out
