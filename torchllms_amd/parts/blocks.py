"""Arrangements of a layer's parts."""

from __future__ import annotations

from .base import BLOCKS, Block


@BLOCKS.register("pre_norm")
class PreNormBlock(Block):
    """``h = x + mixer(norm(x)); out = h + ffn(norm(h))``
    (reference: torchllms/models/networks.py:635-644).  Each residual sum is fused into the
    norm that reads it; the last one is handed on as ``delta``."""

    graph_safe = True
    SLOTS = {"mixer_norm": "norm", "mixer": "mixer", "ffn_norm": "norm", "ffn": "feed_forward"}

    def forward(self, h, delta, ctx, cache):
        h, y = self.mixer_norm.forward_add_for(self.mixer, h, delta)
        a = self.mixer.forward(y, ctx, cache["mixer"])
        h, y = self.ffn_norm.forward_add_for(self.ffn, h, a)
        f = self.ffn.forward(y, ctx)
        return h, f
