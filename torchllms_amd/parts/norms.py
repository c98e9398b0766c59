"""Normalisations."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import NORMS, Norm, ParamSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    """``y = cast(x32 * rsqrt(mean(x32^2) + eps)) * weight``: statistics and scaling in 32-bit,
    the weight multiply after the cast back (reference: torchllms/models/networks.py:186-200)."""

    graph_safe = True
    takes_split_sums = True  # ops.rmsnorm adds the slices of a split product while it reads them

    def __init__(self, size: int, eps: float):
        self.size = size
        self.eps = float(eps)
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.size,), kind="vector", init="ones")}

    def check_sizes(self, dtype: torch.dtype) -> None:
        if not 0 < self.size <= ops.rmsnorm_max_hidden():
            raise ValueError(f"rmsnorm: rows of {self.size} elements; the kernel takes 1 to {ops.rmsnorm_max_hidden()}")

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors["weight"].contiguous()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(x, self.weight, self.eps)

    def forward_add(self, h: torch.Tensor, delta: Optional[torch.Tensor]):
        if delta is None:
            return h, ops.rmsnorm(h, self.weight, self.eps)
        return ops.rmsnorm(h, self.weight, self.eps, delta=delta, return_sum=True)

    def forward_add_for(self, reader, h: torch.Tensor, delta):
        if (isinstance(delta, ops.PendingProduct) and getattr(reader, "takes_normed_rows", False)
                and self.weight.dtype == torch.bfloat16 and self.size <= ops.NORMED_ROWS_MAX_WIDTH):
            # the product's own kernel adds it to h and leaves the rows' statistics, which the reader's kernel applies
            return delta.added_to(h, self.weight, self.eps)
        return self.forward_add(h, delta)

    def forward_rows(self, h: torch.Tensor, delta: Optional[torch.Tensor], rows: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(h, self.weight, self.eps, delta=delta, rows=rows)
