"""Grouped-query attention over paged keys and values."""

from __future__ import annotations

import logging
from typing import Dict, Optional

import torch

from ..config.spec import PartSpec
from ..kernels import ops
from ..kernels.attention import paged_attention
from .base import MIXERS, POSITIONS, KVNeed, Mixer, ParamSpec


#: (heads, kv heads, head size) whose fall to the plain attention kernel has been reported
_SAID_SLOW: set = set()


@MIXERS.register("attention")
class Attention(Mixer):
    """q/k/v projections, position encoding on q and k, keys and values appended to the cache,
    causal attention of the new queries over everything cached for their request, output
    projection (reference: torchllms/models/networks.py:460-558; plain formula 355-397).

    Query head h reads key/value head ``h // (num_heads / num_kv_heads)``.  ``window`` w > 0
    limits a query at position p to keys p-w+1..p.  ``shares_kv``: this layer has no k/v
    projections and reads the cache of the run named by the execution order.  ``kv_page_size``:
    tokens per page of this layer's keys and values, when not the engine's own (layers that ask for
    the same form a group of pages of their own).
    """

    #: every launch is fixed by the step's shape: a decode step may be recorded in a HIP graph
    graph_safe = True
    takes_normed_rows = True

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        qkv_bias: bool,
        softmax_scale: float,
        window: int,
        position: PartSpec,
        shares_kv: bool = False,
        kv_page_size: Optional[int] = None,
    ):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.qkv_bias = qkv_bias
        self.softmax_scale = float(softmax_scale)
        self.window = int(window)
        self.shares_kv = shares_kv
        self.kv_page_size = kv_page_size
        self.position = POSITIONS.build(position)
        self.wqkv: Optional[torch.Tensor] = None
        self.bqkv: Optional[torch.Tensor] = None
        self.wo: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        q = self.num_heads * self.head_dim
        kv = self.num_kv_heads * self.head_dim
        specs = {"wq.weight": ParamSpec((q, self.hidden_size)), "wo.weight": ParamSpec((self.hidden_size, q))}
        if not self.shares_kv:
            specs["wk.weight"] = ParamSpec((kv, self.hidden_size))
            specs["wv.weight"] = ParamSpec((kv, self.hidden_size))
        if self.qkv_bias:
            specs["wq.bias"] = ParamSpec((q,), init="zeros")
            if not self.shares_kv:
                specs["wk.bias"] = ParamSpec((kv,), init="zeros")
                specs["wv.bias"] = ParamSpec((kv,), init="zeros")
        return specs

    def check_sizes(self, dtype: torch.dtype) -> None:
        if not 0 < self.head_dim <= ops.ATTENTION_MAX_HEAD_DIM:
            raise ValueError(
                f"attention: head size {self.head_dim}; the attention kernels take head sizes up to "
                f"{ops.ATTENTION_MAX_HEAD_DIM} (any number of heads and of query heads per kv head)"
            )
        if dtype == torch.bfloat16:
            fast = (ops.decode_attention_supported(dtype, self.num_heads, self.num_kv_heads, self.head_dim),
                    ops.prefill_attention_supported(dtype, self.num_heads, self.num_kv_heads, self.head_dim))
            said = (self.num_heads, self.num_kv_heads, self.head_dim)
            if not all(fast) and said not in _SAID_SLOW:
                _SAID_SLOW.add(said)
                logging.getLogger("torchllms_amd").warning(
                    "attention with %d heads in %d groups of head size %d: the matrix-core kernels take head sizes %s with at "
                    "most 16 query heads per kv head (8 at head size 256 in decode steps); %s run the plain kernel (right, and several times slower)",
                    self.num_heads, self.num_kv_heads, self.head_dim, "/".join(str(d) for d in ops.DECODE_HEAD_DIMS),
                    "decode steps and prompts" if not any(fast) else "decode steps" if not fast[0] else "prompts",
                )
        rot = self.position.rotary_args()
        if rot is not None and (rot.rotary_dim % 2 or rot.rotary_dim > self.head_dim):
            raise ValueError(f"attention: {rot.rotary_dim} rotated channels of a head of {self.head_dim} (even, at most the head size)")

    def cache_need(self):
        if self.shares_kv:
            return None
        return KVNeed(num_kv_heads=self.num_kv_heads, head_dim=self.head_dim, window=self.window, page_size=self.kv_page_size)

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        names = ["wq"] if self.shares_kv else ["wq", "wk", "wv"]
        # one fused projection [q rows | k rows | v rows]: a single matrix product per token batch
        self.wqkv = torch.cat([tensors[f"{n}.weight"] for n in names], dim=0).contiguous()
        if self.qkv_bias:
            self.bqkv = torch.cat([tensors[f"{n}.bias"] for n in names], dim=0).contiguous()
        self.wo = tensors["wo.weight"].contiguous()
        self.position.to(self.wo.device)

    def linear_weights(self):
        return [(self.wqkv, "qkv"), (self.wo, "sum")]

    def forward(self, x, ctx, cache):
        n_kv_in_row = 0 if self.shares_kv else self.num_kv_heads
        rot = self.position.rotary_args()
        g = cache.group
        store = cache.writes and not self.shares_kv
        # cosines and sines of this step's positions: made once per step and shared by every layer
        # whose position encoding has the same frequencies
        table = None
        if rot is not None and rot.rotary_dim > 0:
            key = ("rope_table", rot.inv_freq.data_ptr())
            table = ctx.scratch.get(key)
            if table is None:
                table = ctx.scratch[key] = ops.rope_table(ctx.positions, rot.inv_freq)
        qkv = ops.qkv_rope_store(
            x,
            self.wqkv,
            self.bqkv,
            self.num_heads,
            n_kv_in_row,
            self.head_dim,
            ctx.positions,
            rot.inv_freq if rot else None,
            rot.rotary_dim if rot else 0,
            rot.pairing if rot else 0,
            table,
            cache.k_pages if store else None,
            cache.v_pages if store else None,
            ctx.slot_mappings[g] if store else None,
            cache.page_size if store else 0,
        )
        attn = paged_attention(
            qkv, self.num_heads, self.num_kv_heads, self.head_dim, cache.k_pages, cache.v_pages,
            ctx, g, self.window, self.softmax_scale,
        )
        return ops.linear_to_sum(attn, self.wo, may_wait=True)
