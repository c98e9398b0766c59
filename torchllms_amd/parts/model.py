"""Puts a model together from a ``ModelSpec`` and runs it over one step's tokens."""

from __future__ import annotations

from typing import Dict, List, Tuple

import torch

from ..config.spec import ModelSpec
from .base import BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, Block, ParamSpec

# importing the modules registers the built-in parts
from . import attention as _attention  # noqa: F401
from . import blocks as _blocks  # noqa: F401
from . import embedding as _embedding  # noqa: F401
from . import feed_forward as _feed_forward  # noqa: F401
from . import norms as _norms  # noqa: F401
from . import positions as _positions  # noqa: F401


class Model:
    """Embedding, layers in the order the spec lists, final norm, output head.

    Tensor names: ``embed.weight``, ``<layer name>.<slot>.<param>`` with slots ``mixer_norm``,
    ``mixer``, ``ffn_norm``, ``ffn``, then ``final_norm.weight`` and ``head.weight``.
    """

    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.embedding = EMBEDDINGS.build(spec.embedding)
        self.blocks: List[Block] = []
        for layer in spec.layers:
            block_cls = BLOCKS[layer.block] if layer.block in BLOCKS else None
            if block_cls is None:
                raise KeyError(f"no block arrangement named {layer.block!r}; registered: {sorted(BLOCKS)}")
            self.blocks.append(
                block_cls(
                    mixer=MIXERS.build(layer.mixer),
                    feed_forward=FEED_FORWARDS.build(layer.feed_forward),
                    mixer_norm=NORMS.build(layer.mixer_norm),
                    ffn_norm=NORMS.build(layer.ffn_norm),
                )
            )
        self.final_norm = NORMS.build(spec.final_norm)
        self.head = HEADS.build(spec.head)
        self.dtype = None
        self.device = None

    # ------------------------------------------------------------------ tensors
    def param_specs(self) -> Dict[str, ParamSpec]:
        out: Dict[str, ParamSpec] = {}
        for name, spec in self.embedding.param_specs().items():
            out[f"embed.{name}"] = spec
        for layer, block in zip(self.spec.layers, self.blocks):
            for name, spec in block.param_specs().items():
                out[f"{layer.name}.{name}"] = spec
        for name, spec in self.final_norm.param_specs().items():
            out[f"final_norm.{name}"] = spec
        for name, spec in self.head.param_specs().items():
            out[f"head.{name}"] = spec
        return out

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Hand every part its tensors (already on the device, in their final dtypes)."""

        def sub(prefix: str) -> Dict[str, torch.Tensor]:
            prefix = prefix + "."
            return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}

        self.embedding.bind(sub("embed"))
        for layer, block in zip(self.spec.layers, self.blocks):
            block.bind(sub(layer.name))
        self.final_norm.bind(sub("final_norm"))
        self.head.bind(sub("head"))
        if getattr(self.head, "tied", False):
            self.head.tie(self.embedding)
        emb = tensors["embed.weight"]
        self.dtype = emb.dtype
        self.device = emb.device

    def linear_weights(self):
        """All matrices of the model, grouped by (shape, use): see ``Part.linear_weights``."""
        groups = {}
        parts = [self.head]
        for b in self.blocks:
            parts += [b.mixer, b.feed_forward]
        for part in parts:
            for item in part.linear_weights():
                w, use = item if isinstance(item, tuple) else (item, "plain")
                if w is not None:
                    groups.setdefault((tuple(w.shape), use), []).append(w)
        return groups

    # ------------------------------------------------------------------ cache
    def cache_needs(self) -> List[Tuple[int, object]]:
        """``(run id, need)`` for every run that owns a cache entry."""
        needs = []
        for run_id, run in enumerate(self.spec.order):
            if run.cache_from is not None:
                continue
            needs.append((run_id, self.blocks[run.layer].mixer.cache_need()))
        return needs

    # ------------------------------------------------------------------ one step
    def forward(self, ctx, cache) -> torch.Tensor:
        """Run this step's tokens; returns float32 logits [len(ctx.logit_rows), vocab]."""
        h = self.embedding.forward(ctx.tokens)
        delta = None
        for run_id, run in enumerate(self.spec.order):
            view = cache.view_for_run(run_id, run.cache_from)
            h, delta = self.blocks[run.layer].forward(h, delta, ctx, view)
        if ctx.logit_rows.numel() == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=h.device)
        x = self.final_norm.forward_rows(h, self.final_norm.delta(delta), ctx.logit_rows)
        return self.head.forward(x)
