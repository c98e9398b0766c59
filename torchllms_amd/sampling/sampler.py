"""Chooses next tokens from a step's logits with the sampling kernel."""

from __future__ import annotations

from typing import List, Sequence

import torch

from ..kernels import ops
from .params import SamplingParams


class Sampler:
    """``sampler(logits, params, steps)`` -> one token id per row.

    Row i is drawn with ``params[i]`` at generator counter ``steps[i]`` (the number of tokens the
    request has generated so far), so the same request gives the same tokens whatever else is in
    the batch and however often it was preempted.
    """

    def __init__(self):
        # the tensors of the last batch's parameters: a generation loop asks with the same
        # requests step after step, and only the counters change
        self._key = None
        self._fixed = None
        # the counters travel through a pinned buffer with an asynchronous copy, so that the sampling
        # kernel is queued behind the step's kernels without the host waiting in between; the buffer
        # is free again once the previous call's result has been read (its .tolist() waits)
        self._pinned = None
        self._counters = None

    def __call__(self, logits: torch.Tensor, params: Sequence[SamplingParams], steps: Sequence[int]) -> List[int]:
        return self.launch(logits, params, steps).tolist()

    def launch(self, logits: torch.Tensor, params: Sequence[SamplingParams], steps: Sequence[int], out: torch.Tensor = None) -> torch.Tensor:
        """Queue the sampling behind the step's kernels and return the token ids as a tensor on the
        device: the host goes on until it asks for them (``.tolist()``), which it has to do before
        the next call.  ``out``: where on the device the token ids are to go (int32, one per row)."""
        n = logits.shape[0]
        if n == 0:
            return torch.empty((0,), dtype=torch.int32)
        if len(params) != n or len(steps) != n:
            raise ValueError("one SamplingParams and one step counter per logits row")
        dev = logits.device
        key = (dev, tuple((p.temperature, p.seed, p.top_k) for p in params))
        if key != self._key:
            temperature = torch.tensor([p.temperature for p in params], dtype=torch.float32, device=dev)
            seeds = torch.tensor([_as_i64(p.seed) for p in params], dtype=torch.int64, device=dev)
            top_k = None
            if any(p.top_k for p in params):
                top_k = torch.tensor([p.top_k or 0 for p in params], dtype=torch.int32, device=dev)
            self._key, self._fixed = key, (temperature, seeds, top_k)
        temperature, seeds, top_k = self._fixed
        if self._counters is not None and self._counters.device == dev and self._counters.numel() >= n and all(p.temperature == 0 for p in params):
            # greedy rows draw nothing: the counters are not read, so none are sent
            return ops.sample(logits, temperature, seeds, self._counters[:n], top_k, out=out)
        if self._pinned is None or self._pinned.numel() < n or self._counters.device != dev:
            self._pinned = torch.empty((max(n, 64),), dtype=torch.int64, pin_memory=True)
            self._counters = torch.empty((max(n, 64),), dtype=torch.int64, device=dev)
        self._pinned[:n] = torch.as_tensor([int(s) for s in steps], dtype=torch.int64)
        counters = self._counters[:n]
        counters.copy_(self._pinned[:n], non_blocking=True)
        return ops.sample(logits, temperature, seeds, counters, top_k, out=out)


def _as_i64(x: int) -> int:
    """A seed of up to 64 bits as the signed integer with the same bits."""
    x &= (1 << 64) - 1
    return x - (1 << 64) if x >= (1 << 63) else x
