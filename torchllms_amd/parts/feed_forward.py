"""Feed-forward networks."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import FEED_FORWARDS, FeedForward, ParamSpec


@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    """``w2( silu(w1 x) * (w3 x) )`` without biases
    (reference: torchllms/models/networks.py:592-605)."""

    graph_safe = True
    takes_normed_rows = True

    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.w13: Optional[torch.Tensor] = None
        self.w2: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        f, d = self.intermediate_size, self.hidden_size
        return {"w1.weight": ParamSpec((f, d)), "w3.weight": ParamSpec((f, d)), "w2.weight": ParamSpec((d, f))}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        # gate and up projections fused into one [2F, D] matrix: one product, then silu(gate) * up
        self.w13 = torch.cat([tensors["w1.weight"], tensors["w3.weight"]], dim=0).contiguous()
        self.w2 = tensors["w2.weight"].contiguous()

    def linear_weights(self):
        return [(self.w13, "glu"), (self.w2, "sum")]

    def forward(self, x, ctx):
        return ops.linear_to_sum(ops.linear_glu(x, self.w13), self.w2, may_wait=True)
