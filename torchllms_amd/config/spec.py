"""Architecture-neutral description of a model: which parts, with which sizes, in which order.

A ``ModelSpec`` is pure data.  An architecture's builder turns its typed configuration into
one; the engine turns a ``ModelSpec`` into live parts by looking every ``PartSpec.kind`` up
in the part registries.  Nothing here knows a concrete architecture.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


@dataclass(frozen=True)
class PartSpec:
    """One part: ``kind`` is a key of the matching part registry, ``params`` are the
    keyword arguments of that part's constructor (all sizes and constants)."""

    kind: str
    params: Dict[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """One layer = an arrangement (``block``, a key of the block registry) and the parts it arranges.

    ``parts`` maps the arrangement's slot names to parts.  Which slots there are, and which kind of
    part each takes (mixer, feed-forward, norm), is the arrangement's own business: a pre-norm
    block has ``mixer_norm``, ``mixer``, ``ffn_norm`` and ``ffn``; one with norms on both sides of
    every branch has six; one without a feed-forward has two.  ``block_params`` are further keyword
    arguments of the arrangement (a residual scale, say).
    ``name`` is the prefix of the layer's tensors inside the model ("layers.3"); a sub-part's
    tensors follow as ``<name>.<slot>.<tensor>``.
    """

    name: str
    block: str
    parts: Dict[str, PartSpec]
    block_params: Dict[str, Any] = field(default_factory=dict)


def standard_layer(name: str, block: str, mixer: PartSpec, feed_forward: PartSpec, mixer_norm: PartSpec,
                   ffn_norm: PartSpec, **block_params: Any) -> LayerSpec:
    """A layer of the common four parts under their usual slot names."""
    return LayerSpec(
        name=name,
        block=block,
        parts={"mixer_norm": mixer_norm, "mixer": mixer, "ffn_norm": ffn_norm, "ffn": feed_forward},
        block_params=dict(block_params),
    )


@dataclass(frozen=True)
class LayerRun:
    """One entry of the execution order.

    ``layer`` indexes ``ModelSpec.layers`` (a layer may appear in several runs and then
    shares its weights between them).  Every run owns a cache entry of its own unless
    ``cache_from`` names an earlier run: then this run reads that run's cache and writes none.
    """

    layer: int
    cache_from: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec
    layers: List[LayerSpec]
    order: List[LayerRun]
    final_norm: PartSpec
    head: PartSpec

    def validate(self) -> None:
        n = len(self.layers)
        for i, run in enumerate(self.order):
            if not 0 <= run.layer < n:
                raise ValueError(f"order[{i}] names layer {run.layer}, but the model has {n} layers")
            if run.cache_from is not None:
                if not 0 <= run.cache_from < i:
                    raise ValueError(
                        f"order[{i}].cache_from={run.cache_from} must name an earlier run (0..{i - 1})"
                    )
                if self.order[run.cache_from].cache_from is not None:
                    raise ValueError(
                        f"order[{i}].cache_from={run.cache_from} names a run that itself borrows a cache"
                    )
