"""Token embedding and output head."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import EMBEDDINGS, HEADS, Embedding, Head, ParamSpec


@EMBEDDINGS.register("embedding")
class TokenEmbedding(Embedding):
    """``h = weight[token]``, no scale factor (reference: torchllms/models/networks.py:793,1017)."""

    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.vocab_size, self.hidden_size))}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors["weight"].contiguous()

    def forward(self, tokens: torch.Tensor) -> torch.Tensor:
        return ops.embed(tokens, self.weight)


@HEADS.register("lm_head")
class LMHead(Head):
    """``logits = x W^T`` with W [vocab, hidden], no bias; with ``tied`` W is the embedding
    matrix (reference: torchllms/models/networks.py:804-809,1047).  Logits are returned in 32-bit."""

    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool):
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.tied = tied
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        if self.tied:
            return {}
        return {"weight": ParamSpec((self.vocab_size, self.hidden_size))}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        if not self.tied:
            self.weight = tensors["weight"].contiguous()

    def tie(self, embedding: TokenEmbedding) -> None:
        self.weight = embedding.weight

    def linear_weights(self):
        return [(self.weight, "plain", torch.float32)]

    def ignorable_params(self):
        # checkpoints of tied models sometimes carry the output matrix all the same
        return ["weight"] if self.tied else []

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.linear(x, self.weight, out_dtype=torch.float32)
