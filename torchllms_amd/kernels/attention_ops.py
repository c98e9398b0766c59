"""Attention over the paged cache: the plain kernel (any size, both dtypes), the split-KV decode kernel and
the tiled prefill kernel (bfloat16, MFMA), with the host-side plans of their launches."""

from __future__ import annotations

from typing import Optional

import torch

from .base import (  # noqa: F401
    BF16,
    F32,
    KernelError,
    SplitSums,
    _gpu,
    _i32,
    _ptr,
    _stream,
    check,
    core,
    device_facts,
    dtype_code,
    resolved,
    variant,
)


#: the largest head size any attention kernel here takes (the plain kernel's; the MFMA kernels take
#: ``DECODE_HEAD_DIMS`` / ``PREFILL_HEAD_DIMS``, everything else below this runs the plain kernel)
ATTENTION_MAX_HEAD_DIM = 256


def _generic_arguments(qkv, n_q_heads, n_kv_heads, head_dim, k_pages, v_pages, token_seq, positions, block_table, out):
    """What both launches of the plain kernel ask of their arguments; returns (tokens, page size, out)."""
    _gpu(qkv, k_pages, v_pages, token_seq, positions, block_table)
    _i32(token_seq, "token_seq")
    _i32(positions, "positions")
    n = qkv.shape[0]
    if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] < n_q_heads * head_dim:
        raise KernelError("attention: qkv must be row-major with at least Hq * dh columns")
    if token_seq.numel() != n or positions.numel() != n:
        raise KernelError("attention: token_seq and positions need one entry per token")
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or block_table.stride(1) != 1:
        raise KernelError("attention: block_table must be an int32 matrix")
    page_size = k_pages.shape[2]
    for pg in (k_pages, v_pages):
        if pg.dim() != 4 or pg.shape[1:] != (n_kv_heads, page_size, head_dim) or pg.dtype != qkv.dtype or not pg.is_contiguous():
            raise KernelError("attention: pages must be contiguous [pages, Hkv, page_size, dh] of the query's dtype")
    if out is None:
        out = torch.empty((n, n_q_heads * head_dim), dtype=qkv.dtype, device=qkv.device)
    return n, page_size, out


def attention_generic(
    qkv: torch.Tensor,
    n_q_heads: int,
    n_kv_heads: int,
    head_dim: int,
    k_pages: torch.Tensor,
    v_pages: torch.Tensor,
    token_seq: torch.Tensor,
    positions: torch.Tensor,
    block_table: torch.Tensor,
    window: int,
    scale: float,
    out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Attention of each token's query heads (the first Hq * dh columns of ``qkv``) over the paged
    keys and values of its request; returns [n, Hq * dh]."""
    n, page_size, out = _generic_arguments(qkv, n_q_heads, n_kv_heads, head_dim, k_pages, v_pages, token_seq, positions, block_table, out)
    check(
        core().tl_attention_generic(
            qkv.data_ptr(), qkv.stride(0), out.data_ptr(), out.stride(0), k_pages.data_ptr(), v_pages.data_ptr(),
            token_seq.data_ptr(), positions.data_ptr(), block_table.data_ptr(), block_table.stride(0), n,
            n_q_heads, n_kv_heads, head_dim, page_size, window, float(scale), dtype_code(qkv.dtype), _stream(),
        )
    )
    return out


# ----------------------------------------------------------------------------- decode attention (bfloat16, MFMA)
_P, _I, _F = __import__("ctypes").c_void_p, __import__("ctypes").c_int, __import__("ctypes").c_float
def attention_generic_split(
    qkv: torch.Tensor,
    n_q_heads: int,
    n_kv_heads: int,
    head_dim: int,
    k_pages: torch.Tensor,
    v_pages: torch.Tensor,
    token_seq: torch.Tensor,
    positions: torch.Tensor,
    block_table: torch.Tensor,
    window: int,
    scale: float,
    longest: int,
    out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """``attention_generic`` for steps with few tokens and long contexts (decode): every block of 64
    keys is computed by a wave of its own and a second kernel joins the blocks in order.  The same
    blocks, operations and order as the one-wave form: the same bits.  ``longest``: an upper bound of
    the keys any token sees (its position + 1, or the window)."""
    n, page_size, out = _generic_arguments(qkv, n_q_heads, n_kv_heads, head_dim, k_pages, v_pages, token_seq, positions, block_table, out)
    # blocks are aligned to absolute positions: a range of `longest` keys touches at most this many
    max_blocks = max(int(longest), 1) // 64 + 2
    partials = torch.empty((n, n_q_heads, max_blocks, head_dim + 2), dtype=torch.float32, device=qkv.device)
    check(
        core().tl_attention_generic_split(
            qkv.data_ptr(), qkv.stride(0), out.data_ptr(), out.stride(0), k_pages.data_ptr(), v_pages.data_ptr(),
            token_seq.data_ptr(), positions.data_ptr(), block_table.data_ptr(), block_table.stride(0), n,
            n_q_heads, n_kv_heads, head_dim, page_size, window, float(scale), dtype_code(qkv.dtype), max_blocks,
            partials.data_ptr(), _stream(),
        )
    )
    return out


_DECODE_SIGNATURES = {
    "tl_attn_decode": [_P, _I, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _I, _I, _P, _P, _P],
}
DECODE_HEAD_DIMS = (32, 64, 128, 256)
_DECODE_BLOCK_KEYS = 64  # keys one block pass covers (4 waves x 16): splits are multiples of it


def decode_attention_supported(dtype: torch.dtype, n_q_heads: int, n_kv_heads: int, head_dim: int) -> bool:
    """Whether the MFMA decode kernel takes these sizes (else the plain kernel runs)."""
    if dtype != torch.bfloat16 or head_dim not in DECODE_HEAD_DIMS or n_q_heads % n_kv_heads:
        return False
    return n_q_heads // n_kv_heads <= (16 if head_dim <= 128 else 8)


_DECODE_MIN_SPLIT = 128  # keys: shorter splits cost more in the merge than they gain in spread (with 256, short contexts at small batches left most CUs idle: one request of 2,176 keys 12.5 -> 10.0 us, eight of 1,024 15.9 -> 14.6)
#: blocks a CU takes at a time before a launch stops gaining from more splits, by head size: about
#: 64 KB of keys and values in flight on a CU (a block's four waves fetch 64 keys and values a pass)
_DECODE_BLOCKS_PER_CU = {32: 3, 64: 3, 128: 2, 256: 1}
#: up to this many (request, kv head) pairs a launch at head size 128 aims at one block a CU: the splits are long
#: then, a CU's one block keeps its loads in flight by itself, and half as many partial results go through the merge
#: (two requests of 8,192 keys: 21.6 -> 20.7 us; one of 16,384: 23.4 -> 21.9, of 32,768: 37.6 -> 32.8; four of 4,096:
#: 21.5 -> 19.6; at head size 64 two and three blocks a CU stayed better at every size)
_DECODE_FEW_PAIRS = 32


#: from this many keys on no split is longer than ``_DECODE_LONGEST_SPLIT``: a launch of few long blocks ends when
#: its slowest block does, and blocks that wait for a free CU even that out (alone, cold, planned -> capped, us: two
#: requests of 32,768 keys 64 -> 55, four 107 -> 98, eight 199 -> 193; sixteen of 8,192 108 -> 101, sixty-four 382 ->
#: 372; sixty-four of 2,176 keys lose 14% when cut, hence the threshold)
_DECODE_LONG = 4096
_DECODE_LONGEST_SPLIT = 1024
DECODE_UNEVEN_SPLIT = 512  # keys: the longest split when requests differ much in length (measured with 64 requests of 128 to 4,608 tokens: 1 to 1.5% more tokens a second than with 1,024, 12% more than with 2,048)


def plan_decode_splits(n_tokens: int, n_kv_heads: int, longest: int, head_dim: int = 128, uneven: bool = False):
    """``(split_size, n_splits)`` for a decode launch whose longest visible key range (counted from
    its 16-aligned start) is ``longest``: as many splits as give every CU its share of blocks and
    no more (two blocks a CU at head size 128, one at 256, three at 64 and 32), none shorter than
    128 keys.  A launch is as long as its most loaded CU, so a few blocks beyond a whole number a CU
    cost as much as a whole further round, and every split costs its start, its partial results
    and its share of the merge; staying under the limit was the best choice or within 1% of it on
    average (at most 11%) over 1 to 100 requests of 700 to 20,000 tokens at each head size, where
    always aiming at 512 blocks lost 3 to 16% on average.  A batch with that many (request, kv
    head) pairs or more is not split at all, if the requests are about equally long and hold fewer than
    4,096 keys; from there on no split is longer than 1,024 keys.

    ``uneven``: the requests differ much in length.  Then all blocks of such a launch would be
    resident at once and stay where they were put, a CU with long requests' blocks working on
    when its neighbours have finished; with splits of at most 512 keys there are several times
    more blocks than fit, and those that wait go where others end.  (64 requests of 128 to 4,608
    tokens: 30% less time than unsplit; 64 equal ones: 10% more, hence the switch.)"""
    pairs = max(n_tokens * n_kv_heads, 1)
    per_cu = _DECODE_BLOCKS_PER_CU.get(head_dim, 2)
    if head_dim == 128 and pairs <= _DECODE_FEW_PAIRS:
        per_cu = 1
    limit = device_facts()[0] * per_cu
    want = max(limit // pairs, 1)
    split = -(-max(longest, 1) // want)
    if longest >= _DECODE_LONG:
        split = min(split, _DECODE_LONGEST_SPLIT)
    if uneven:
        split = min(split, DECODE_UNEVEN_SPLIT)
    split = max(-(-split // _DECODE_BLOCK_KEYS) * _DECODE_BLOCK_KEYS, _DECODE_MIN_SPLIT)
    return split, max(-(-max(longest, 1) // split), 1)


def attention_decode(
    qkv: torch.Tensor,
    n_q_heads: int,
    n_kv_heads: int,
    head_dim: int,
    k_pages: torch.Tensor,
    v_pages: torch.Tensor,
    token_seq: torch.Tensor,
    positions: torch.Tensor,
    block_table: torch.Tensor,
    window: int,
    scale: float,
    longest: int,
    out: Optional[torch.Tensor] = None,
    split_size: Optional[int] = None,
    uneven: bool = False,
) -> torch.Tensor:
    """Attention of single-token queries over their requests' pages with the split-KV MFMA kernel.
    ``longest``: an upper bound of any token's visible key range, counted from its 16-aligned first
    visible key (position + 1 without a window)."""
    _gpu(qkv, k_pages, v_pages, token_seq, positions, block_table)
    _i32(token_seq, "token_seq")
    _i32(positions, "positions")
    if qkv.dtype != torch.bfloat16:
        raise KernelError("attention_decode takes bfloat16")
    n = token_seq.numel()
    if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[0] < n or qkv.shape[1] < n_q_heads * head_dim:
        raise KernelError("attention_decode: qkv must be row-major with a row per token and at least Hq * dh columns")
    if positions.numel() != n:
        raise KernelError("attention_decode: one position per token")
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or block_table.stride(1) != 1:
        raise KernelError("attention_decode: block_table must be an int32 matrix")
    page_size = k_pages.shape[2]
    for pg in (k_pages, v_pages):
        if pg.dim() != 4 or pg.shape[1:] != (n_kv_heads, page_size, head_dim) or pg.dtype != qkv.dtype or not pg.is_contiguous():
            raise KernelError("attention_decode: pages must be contiguous [pages, Hkv, page_size, dh] bfloat16")
    if out is None:
        out = torch.empty((n, n_q_heads * head_dim), dtype=qkv.dtype, device=qkv.device)
    if split_size is None:
        split_size, n_splits = plan_decode_splits(n, n_kv_heads, longest, head_dim, uneven=uneven)
    else:
        n_splits = max(-(-max(longest, 1) // split_size), 1)
    ws_o = ws_ml = None
    if n_splits > 1:
        ws_o = torch.empty((n * n_q_heads * n_splits * head_dim,), dtype=torch.float32, device=qkv.device)
        ws_ml = torch.empty((n * n_q_heads * n_splits * 2,), dtype=torch.float32, device=qkv.device)
    lib = variant("attn_decode", head_dim, _DECODE_SIGNATURES)
    check(
        lib.tl_attn_decode(
            qkv.data_ptr(), qkv.stride(0), out.data_ptr(), out.stride(0), k_pages.data_ptr(), v_pages.data_ptr(),
            token_seq.data_ptr(), positions.data_ptr(), block_table.data_ptr(), block_table.stride(0), n,
            n_q_heads, n_kv_heads, head_dim, page_size, window, float(scale), split_size, n_splits,
            _ptr(ws_o), _ptr(ws_ml), _stream(),
        ),
        lib,
        "tl_variant_last_error",
    )
    return out


# ----------------------------------------------------------------------------- prefill attention (bfloat16, MFMA)
_PREFILL_SIGNATURES = {
    "tl_attn_prefill": [_P, _I, _P, _I, _P, _P, _P, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P],
}
PREFILL_HEAD_DIMS = (32, 64, 128, 256)


def prefill_attention_supported(dtype: torch.dtype, n_q_heads: int, n_kv_heads: int, head_dim: int, page_size: int = 16) -> bool:
    """Whether the MFMA prefill kernel takes these sizes (else the plain kernel runs): bfloat16, head
    size 32, 64, 128 or 256, at most 16 query heads per kv head, pages of a power of two of tokens that
    hold at least the rows a wave fetches with one instruction (1 KB: 512 / head size rows, which then
    share one entry of the block table)."""
    return (dtype == torch.bfloat16 and head_dim in PREFILL_HEAD_DIMS and n_q_heads % n_kv_heads == 0
            and n_q_heads // n_kv_heads <= 16 and page_size > 0 and page_size & (page_size - 1) == 0
            and page_size * head_dim >= 512)


def prefill_queries_per_tile(n_q_heads: int, n_kv_heads: int, head_dim: int) -> int:
    """Queries one block of the prefill kernel covers: its MFMA columns (128, or 64 at head size 256)
    divided by the group size rounded up to a power of two."""
    group = n_q_heads // n_kv_heads
    rp = 1
    while rp < group:
        rp *= 2
    return (128 if head_dim <= 128 else 64) // rp


#: launches of up to this many blocks run with two sets of waves per block, whatever their keys: one block of
#: one set a CU leaves half of every CU idle
PREFILL_SPLIT_ALWAYS = 256
#: launches of up to this many blocks run with two sets of waves while no tile sees more than
#: ``PREFILL_SPLIT_KEYS`` keys: behind a long prefix a block lives long enough for two independent blocks on a
#: CU to overlap better than two sets in step.  Measured with cold caches at head size 128, one set against two
#: (us): 256 blocks 41 / 35 without a prefix, 286 / 215 behind 8,192 keys; 384 blocks 57 / 46 without, 90 / 85
#: behind 1,024, 121 / 123 behind 2,048, 313 / 367 behind 8,192; 512 blocks 75 / 69 without, 108 / 107 behind
#: 1,024, 207 / 227 behind 4,096, 337 / 387 behind 8,192; 768 blocks 117 / 129 without, 578 / 588 behind 8,192;
#: 1,024 blocks 194 / 201.
PREFILL_SPLIT_BLOCKS = 512
PREFILL_SPLIT_KEYS = 3072


def prefill_key_groups(n_tiles: int, n_kv_heads: int, longest_keys: int = 0) -> int:
    """Sets of waves per block of the prefill kernel.  A launch whose blocks all fit the GPU at once
    takes as long as its longest block; with two sets of waves, each with every second tile of keys,
    that block's chain is half as long.  A launch of many more blocks keeps the CUs busy anyway, and
    there two independent blocks on a CU overlap better than two sets of waves in step.
    ``longest_keys``: the most keys any tile of the launch sees."""
    blocks = n_tiles * n_kv_heads
    if blocks <= PREFILL_SPLIT_ALWAYS:
        return 2
    return 2 if blocks <= PREFILL_SPLIT_BLOCKS and longest_keys <= PREFILL_SPLIT_KEYS else 1


def prefill_tile_count(qo_indptr, first_row: int, n_rows: int, queries_per_tile: int) -> int:
    return sum(-(-(int(qo_indptr[r + 1]) - int(qo_indptr[r])) // queries_per_tile) for r in range(first_row, n_rows))


def prefill_tiles(qo_indptr, first_row: int, n_rows: int, queries_per_tile: int, kv_lens=None, window: int = 0):
    """Host lists ``(tile_row, tile_q0)`` that cut rows ``first_row .. n_rows-1`` into query tiles.

    With ``kv_lens`` the tiles are put in the order that balances the launch: a tile's cost is the
    number of keys it sees, and late tiles of a causal prompt see many times more than early ones.
    Blocks are handed to the CUs in launch order; longest first lets the short ones fill the gaps at
    the end.  (For launches that about fit the GPU at once an order that puts a long and a short tile
    on every CU was measured too: the same up to 640 blocks, 10% slower at 768, 20% at 1,024.)"""
    rows, q0s, costs = [], [], []
    for r in range(first_row, n_rows):
        q_len = int(qo_indptr[r + 1]) - int(qo_indptr[r])
        pos0 = (int(kv_lens[r]) - q_len) if kv_lens is not None else 0
        for q0 in range(0, q_len, queries_per_tile):
            rows.append(r)
            q0s.append(q0)
            hi = pos0 + min(q0 + queries_per_tile, q_len) - 1
            lo = max(pos0 + q0 - window + 1, 0) if window > 0 else 0
            costs.append(hi - lo + 1)
    if kv_lens is None or len(rows) < 2:
        return rows, q0s
    order = sorted(range(len(rows)), key=lambda i: -costs[i])
    return [rows[i] for i in order], [q0s[i] for i in order]


def attention_prefill(
    qkv: torch.Tensor,
    n_q_heads: int,
    n_kv_heads: int,
    head_dim: int,
    k_pages: torch.Tensor,
    v_pages: torch.Tensor,
    qo_indptr: torch.Tensor,
    kv_lens: torch.Tensor,
    block_table: torch.Tensor,
    tile_row: torch.Tensor,
    tile_q0: torch.Tensor,
    window: int,
    scale: float,
    out: torch.Tensor,
    key_groups: int = 1,
) -> torch.Tensor:
    """Causal attention of the rows named by the tile lists (see ``prefill_tiles``) with the MFMA
    prefill kernel.  Token t of ``qkv`` / ``out`` is token t of ``qo_indptr``'s numbering.
    ``key_groups`` = 2: two sets of waves per block share a tile's keys between them."""
    _gpu(qkv, k_pages, v_pages, qo_indptr, kv_lens, block_table, tile_row, tile_q0, out)
    for t, what in ((qo_indptr, "qo_indptr"), (kv_lens, "kv_lens"), (tile_row, "tile_row"), (tile_q0, "tile_q0")):
        _i32(t, what)
    if qkv.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise KernelError("attention_prefill takes bfloat16")
    if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] < n_q_heads * head_dim:
        raise KernelError("attention_prefill: qkv must be row-major with at least Hq * dh columns")
    if out.dim() != 2 or out.stride(1) != 1 or out.shape[0] != qkv.shape[0] or out.shape[1] < n_q_heads * head_dim:
        raise KernelError("attention_prefill: out must be row-major [tokens, >= Hq * dh]")
    if tile_row.numel() != tile_q0.numel():
        raise KernelError("attention_prefill: tile lists differ in length")
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or block_table.stride(1) != 1:
        raise KernelError("attention_prefill: block_table must be an int32 matrix")
    if kv_lens.numel() != block_table.shape[0] or qo_indptr.numel() != kv_lens.numel() + 1:
        raise KernelError("attention_prefill: qo_indptr, kv_lens and block_table disagree about the rows")
    page_size = k_pages.shape[2]
    for pg in (k_pages, v_pages):
        if pg.dim() != 4 or pg.shape[1:] != (n_kv_heads, page_size, head_dim) or pg.dtype != qkv.dtype or not pg.is_contiguous():
            raise KernelError("attention_prefill: pages must be contiguous [pages, Hkv, page_size, dh] bfloat16")
    lib = variant("attn_prefill", head_dim, _PREFILL_SIGNATURES)
    check(
        lib.tl_attn_prefill(
            qkv.data_ptr(), qkv.stride(0), out.data_ptr(), out.stride(0), k_pages.data_ptr(), v_pages.data_ptr(),
            qo_indptr.data_ptr(), kv_lens.data_ptr(), block_table.data_ptr(), block_table.stride(0),
            tile_row.data_ptr(), tile_q0.data_ptr(), tile_row.numel(), n_q_heads, n_kv_heads, head_dim, page_size,
            window, float(scale), int(key_groups), _stream(),
        ),
        lib,
        "tl_variant_last_error",
    )
    return out
