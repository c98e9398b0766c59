"""Puts a model together from a ``ModelSpec`` and runs it over one step's tokens."""

from __future__ import annotations

from typing import Dict, List, Tuple

import torch

from ..config.spec import ModelSpec
from .base import BLOCKS, EMBEDDINGS, HEADS, NORMS, SLOT_KINDS, Block, ParamSpec, Part

# importing the modules registers the built-in parts
from . import attention as _attention  # noqa: F401
from . import blocks as _blocks  # noqa: F401
from . import embedding as _embedding  # noqa: F401
from . import feed_forward as _feed_forward  # noqa: F401
from . import norms as _norms  # noqa: F401
from . import positions as _positions  # noqa: F401


class Model:
    """Embedding, layers in the order the spec lists, final norm, output head.

    Tensor names: ``embed.<tensor>``, ``<layer name>.<slot>.<tensor>`` with the slots of the layer's
    block arrangement (``mixer_norm``, ``mixer``, ``ffn_norm``, ``ffn`` for a pre-norm block), then
    ``final_norm.<tensor>`` and ``head.<tensor>``.
    """

    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.embedding = EMBEDDINGS.build(spec.embedding)
        self.blocks: List[Block] = []
        for layer in spec.layers:
            if layer.block not in BLOCKS:
                raise KeyError(f"no block arrangement named {layer.block!r}; registered: {sorted(BLOCKS)}")
            block_cls = BLOCKS[layer.block]
            missing = [s for s in block_cls.SLOTS if s not in layer.parts]
            extra = [s for s in layer.parts if s not in block_cls.SLOTS]
            if missing or extra:
                raise ValueError(
                    f"{layer.name}: the arrangement {layer.block!r} has the parts {list(block_cls.SLOTS)}; "
                    f"the layer lacks {missing} and names {extra} that the arrangement does not have"
                )
            parts = {slot: SLOT_KINDS[kind].build(layer.parts[slot]) for slot, kind in block_cls.SLOTS.items()}
            self.blocks.append(block_cls(parts, **layer.block_params))
        self.final_norm = NORMS.build(spec.final_norm)
        self.head = HEADS.build(spec.head)
        # per run: (slot of a mixer, key of its cache entry, whether the run owns the entry)
        self._run_caches: List[List[Tuple[str, Tuple[int, str], bool]]] = []
        for run_id, run in enumerate(spec.order):
            src = run_id if run.cache_from is None else run.cache_from
            if run.cache_from is not None:
                theirs = set(self.blocks[spec.order[src].layer].mixers())
                mine = set(self.blocks[run.layer].mixers())
                if not mine <= theirs:
                    raise ValueError(
                        f"order[{run_id}] borrows the cache of order[{src}], whose layer has no mixer in the "
                        f"slots {sorted(mine - theirs)}"
                    )
            self._run_caches.append([(slot, (src, slot), run.cache_from is None) for slot in self.blocks[run.layer].mixers()])

    def all_parts(self) -> List[Part]:
        """Every part of the model, blocks and their sub-parts included."""
        parts: List[Part] = [self.embedding, self.final_norm, self.head]
        for b in self.blocks:
            parts.append(b)
            parts.extend(b.sub_parts().values())
        return parts

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

    def ignorable_tensors(self) -> List[str]:
        """Names a checkpoint may hold without the model using them (``Part.ignorable_params``)."""
        out = [f"embed.{n}" for n in self.embedding.ignorable_params()]
        for layer, block in zip(self.spec.layers, self.blocks):
            for slot, part in block.sub_parts().items():
                out += [f"{layer.name}.{slot}.{n}" for n in part.ignorable_params()]
        out += [f"final_norm.{n}" for n in self.final_norm.ignorable_params()]
        out += [f"head.{n}" for n in self.head.ignorable_params()]
        return out

    def linear_weights(self):
        """All matrices of the model, grouped by (shape, use, result dtype or None): see
        ``Part.linear_weights``."""
        groups = {}
        for part in self.all_parts():
            for item in part.linear_weights():
                item = item if isinstance(item, tuple) else (item,)
                w = item[0]
                use = item[1] if len(item) > 1 else "plain"
                out_dtype = item[2] if len(item) > 2 else None
                if w is not None:
                    groups.setdefault((tuple(w.shape), use, out_dtype), []).append(w)
        return groups

    def check_sizes(self, dtype: torch.dtype) -> None:
        """Every part says whether kernels exist for its sizes (``Part.check_sizes``)."""
        for part in self.all_parts():
            part.check_sizes(dtype)

    # ------------------------------------------------------------------ cache
    def cache_needs(self) -> List[Tuple[Tuple[int, str], object]]:
        """``((run id, slot), need)`` for every mixer of every run that owns a cache entry."""
        needs = []
        for run_id, run in enumerate(self.spec.order):
            if run.cache_from is not None:
                continue
            for slot, mixer in self.blocks[run.layer].mixers().items():
                needs.append(((run_id, slot), mixer.cache_need()))
        return needs

    # ------------------------------------------------------------------ one step
    def forward(self, ctx, cache) -> torch.Tensor:
        """Run this step's tokens; returns float32 logits [len(ctx.logit_rows), vocab]."""
        h = self.embedding.forward(ctx.tokens)
        delta = None
        for run, entries in zip(self.spec.order, self._run_caches):
            views = {slot: cache.view(key, writes) for slot, key, writes in entries}
            h, delta = self.blocks[run.layer].forward(h, delta, ctx, views)
        if ctx.logit_rows.numel() == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=h.device)
        x = self.final_norm.forward_rows(h, self.final_norm.delta(delta), ctx.logit_rows)
        return self.head.forward(x)
