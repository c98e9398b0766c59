"""Interfaces and registries of the parts a model is put together from.

A part is built from its ``PartSpec.params`` alone: it is told its sizes and constants and
never learns which model it sits in.  These registries hold them:

======================  ==========================================================
``MIXERS``              token mixers (attention, anything with state of its own)
``FEED_FORWARDS``       per-token feed-forward networks (dense or routed)
``NORMS``               normalisations
``POSITIONS``           position encodings used inside a mixer
``BLOCKS``              arrangements of mixer / feed-forward / norms in one layer
``EMBEDDINGS``          token id -> vector
``HEADS``               vector -> logits
======================  ==========================================================

A part declares its tensors with ``param_specs()`` (names local to the part) and receives
them, already on the device and in their final dtype, through ``bind()``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional, Tuple

import torch

from ..config.spec import PartSpec


@dataclass(frozen=True)
class ParamSpec:
    """One tensor a part expects.

    ``kind``: "matrix" (kept in the model's compute dtype), "vector" (compute dtype, but a
    tensor stored in 32-bit stays in 32-bit), "int" (an integer table, kept as int32).
    ``init``: how the random-weights mode fills it: "normal" N(0, 0.02), "ones", "zeros".
    """

    shape: Tuple[int, ...]
    kind: str = "matrix"
    init: str = "normal"


@dataclass(frozen=True)
class KVNeed:
    """A mixer that keeps keys and values of past tokens in pages.

    ``window`` = 0: every past token stays visible.  ``window`` = w > 0: a token at position p
    sees positions p-w+1 .. p only, so pages that lie wholly before that may be given back.
    ``page_size`` (tokens per page) and ``dtype`` ("float32", "bfloat16") are the engine's own
    unless the mixer asks for others; layers that ask for the same form one group of pages.
    """

    num_kv_heads: int
    head_dim: int
    window: int = 0
    page_size: Optional[int] = None
    dtype: Optional[str] = None


@dataclass(frozen=True)
class StateNeed:
    """A mixer that keeps state of fixed size per request (one row per request slot)."""

    shape: Tuple[int, ...]
    dtype: str = "float32"


class Part:
    """Base of all parts."""

    #: True if the part's ``forward`` also takes ``kernels.ops.NormedRows`` in place of its input tensor
    #: (a norm whose statistics are known but not applied): it passes them to ``ops.linear_glu`` or
    #: ``ops.qkv_rope_store``, which apply them on the way, or makes a tensor of them with ``ops.resolved``
    takes_normed_rows = False

    #: True only if what the part launches depends on the step's shape alone (no value read back
    #: to the host, no launch whose size depends on data): a decode step is replayed from a HIP
    #: graph only when every part of the model says so
    graph_safe = False

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Take ownership of this part's tensors (keys as in ``param_specs``)."""
        if tensors:
            raise ValueError(f"{type(self).__name__} takes no tensors, got {sorted(tensors)}")

    def linear_weights(self):
        """The matrices this part multiplies activations with (for kernel selection by measurement):
        tensors, pairs ``(tensor, use)`` where ``use`` names the fused form of the product that
        the part calls ("glu": ``ops.linear_glu``, "qkv": ``ops.qkv_rope_store``, "sum":
        ``ops.linear_to_sum``), or triples ``(tensor, use, out_dtype)`` when the product's result
        has another dtype than its inputs (32-bit logits)."""
        return []

    def ignorable_params(self):
        """Local names of tensors that a checkpoint may hold for this part although the part, as
        configured, has no use for them (an output matrix beside tied embeddings): the loader drops
        them with a warning instead of calling them unexpected."""
        return []

    def check_sizes(self, dtype: torch.dtype) -> None:
        """Raise (``ValueError`` or a subclass) if no kernel takes this part's sizes in ``dtype``;
        called once when an engine is built, so that a size is refused there and not at the first
        step."""


class Norm(Part):
    """y = norm(x).  ``forward_add`` fuses the residual sum that precedes the norm.

    ``forward_add_for`` is what a block calls: it names the part that will read the norm's output, so a
    norm may leave work to that part's kernels where the part has said that it takes it
    (``Part.takes_normed_rows``).

    A mixer or feed-forward whose last matrix product was split along K may hand its result on as
    ``kernels.ops.SplitSums`` (the slices not yet added) instead of a tensor.  Whoever passes a delta
    to a norm passes it through ``norm.delta(...)`` first: a norm whose kernel adds the slices while it
    reads them sets ``takes_split_sums``; for every other norm they are added up there."""

    takes_split_sums = False

    def delta(self, delta):
        if delta is not None and not isinstance(delta, torch.Tensor) and not self.takes_split_sums:
            return delta.resolve()
        return delta

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def forward_add(self, h: torch.Tensor, delta: Optional[torch.Tensor]):
        """Return ``(h + delta, norm(h + delta))``; ``delta`` may be None."""
        if delta is not None:
            h = h + delta
        return h, self.forward(h)

    def forward_add_for(self, reader: Part, h: torch.Tensor, delta):
        """``forward_add`` for a block: ``delta`` is whatever the part before returned, ``reader`` the
        only part that reads the normed rows."""
        return self.forward_add(h, self.delta(delta))

    def forward_rows(self, h: torch.Tensor, delta: Optional[torch.Tensor], rows: torch.Tensor) -> torch.Tensor:
        """``norm((h + delta)[rows])`` for an int32 index vector ``rows``."""
        idx = rows.long()
        x = h.index_select(0, idx)
        if delta is not None:
            x = x + delta.index_select(0, idx)
        return self.forward(x)


class PositionEncoding(Part):
    """Position information applied to queries and keys inside a mixer."""

    def rotary_args(self):
        """``None`` (queries and keys pass unchanged) or a ``RotaryArgs`` that the fused
        rotate-and-store kernel understands."""
        return None


class FeedForward(Part):
    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        raise NotImplementedError


class Mixer(Part):
    def cache_need(self):
        """``KVNeed``, ``StateNeed`` or None."""
        return None

    def forward(self, x: torch.Tensor, ctx, cache) -> torch.Tensor:
        """``x``: [tokens, hidden] of this step.  ``ctx``: the step's ``StepContext``.
        ``cache``: what the cache manager holds for this run (a ``KVLayerView``, a
        ``StateView`` or None), already pointing at the right layer."""
        raise NotImplementedError


class Block(Part):
    """Arrangement of one layer's parts.  ``SLOTS`` names the sub-parts the arrangement has and the
    kind of each ("mixer", "feed_forward" or "norm"), in the order their tensors are listed; the
    model builds them from the layer's ``LayerSpec.parts`` and hands them over as a dict, and each
    is reachable as an attribute of its slot's name.

    ``forward`` takes the residual stream ``h`` and a pending ``delta`` that has not been added to
    it yet (None for the first layer) and returns the same pair, so the sum can be fused into
    whatever reads it next.  ``cache`` maps the slot of every mixer to what the cache manager holds
    for it in this run (a ``KVLayerView``, a ``StateView`` or None)."""

    SLOTS: Dict[str, str] = {}

    def __init__(self, parts: Dict[str, Part]):
        missing = [s for s in self.SLOTS if s not in parts]
        extra = [s for s in parts if s not in self.SLOTS]
        if missing or extra:
            raise ValueError(
                f"{type(self).__name__} arranges the parts {list(self.SLOTS)}; missing {missing}, not its own {extra}"
            )
        self.parts: Dict[str, Part] = {slot: parts[slot] for slot in self.SLOTS}
        for slot, part in self.parts.items():
            setattr(self, slot, part)

    def sub_parts(self) -> Dict[str, Part]:
        return self.parts

    def mixers(self) -> Dict[str, "Mixer"]:
        """slot -> mixer, for every sub-part that may keep something in the cache."""
        return {slot: part for slot, part in self.parts.items() if isinstance(part, Mixer)}

    def param_specs(self) -> Dict[str, ParamSpec]:
        out = {}
        for slot, part in self.sub_parts().items():
            for name, spec in part.param_specs().items():
                out[f"{slot}.{name}"] = spec
        return out

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for slot, part in self.sub_parts().items():
            prefix = slot + "."
            part.bind({k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)})

    def forward(self, h, delta, ctx, cache):
        raise NotImplementedError


class Registry(dict):
    def __init__(self, what: str):
        super().__init__()
        self.what = what

    def register(self, name: str) -> Callable:
        def deco(cls):
            self[name] = cls
            return cls

        return deco

    def build(self, spec: PartSpec, **extra: Any):
        try:
            cls = self[spec.kind]
        except KeyError:
            raise KeyError(f"no {self.what} named {spec.kind!r}; registered: {sorted(self)}") from None
        return cls(**spec.params, **extra)


class Embedding(Part):
    def forward(self, tokens: torch.Tensor) -> torch.Tensor:
        """int32 token ids [n] -> [n, hidden]."""
        raise NotImplementedError


class Head(Part):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """[n, hidden] -> float32 logits [n, vocab]."""
        raise NotImplementedError


MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
#: the kinds a block's ``SLOTS`` may name, and where parts of each kind are registered
SLOT_KINDS = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS}
POSITIONS = Registry("position encoding")
BLOCKS = Registry("block arrangement")
EMBEDDINGS = Registry("embedding")
HEADS = Registry("output head")
