"""How one request wants its tokens chosen and when it stops."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence


@dataclass
class SamplingParams:
    """``temperature`` 0: greedy.  Otherwise logits / max(temperature, 1e-5), optional ``top_k``
    cut, one draw from the softmax (reference: torchllms/inference/utils.py:25-48).  ``seed``
    makes the draws of this request reproducible and independent of what else runs beside it.
    Generation stops at any of ``stop_token_ids`` (the token is kept) or after
    ``max_new_tokens`` (reference: torchllms/inference/llm.py:489-494,568)."""

    temperature: float = 0.0
    top_k: Optional[int] = None
    max_new_tokens: Optional[int] = None
    stop_token_ids: Sequence[int] = ()
    seed: int = 0

    def __post_init__(self):
        if self.temperature < 0:
            raise ValueError(f"temperature must be >= 0, got {self.temperature}")
        if self.top_k is not None and self.top_k <= 0:
            raise ValueError(f"top_k must be positive, got {self.top_k}")
        if self.max_new_tokens is not None and self.max_new_tokens < 0:
            raise ValueError(f"max_new_tokens must be >= 0, got {self.max_new_tokens}")
        self.stop_token_ids = tuple(int(t) for t in self.stop_token_ids)
