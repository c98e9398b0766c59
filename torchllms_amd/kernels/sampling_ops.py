"""The sampling kernel: greedy, temperature and top-k with a counter-based generator."""

from __future__ import annotations

from typing import Optional

import torch

from .base import (  # noqa: F401
    BF16,
    F32,
    KernelError,
    SplitSums,
    _gpu,
    _i32,
    _ptr,
    _stream,
    check,
    core,
    dtype_code,
    resolved,
    variant,
)


def sample(
    logits: torch.Tensor,
    temperature: torch.Tensor,
    seeds: torch.Tensor,
    steps: torch.Tensor,
    top_k: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """One token per row of float32 ``logits`` [n, vocab]; see csrc/sampling.hip for the rule.  Without
    top-k and with few rows, several blocks share a row (``sample_chunks``); the tokens are the same.
    ``temperature`` float32 [n]; ``seeds``/``steps`` int64 [n] (read as unsigned); ``top_k`` int32 [n].
    ``out``: int32 [n] on the same device to receive the tokens (else a new tensor)."""
    _gpu(logits, temperature, seeds, steps, top_k, out)
    _i32(top_k, "top_k")
    if logits.dim() != 2 or logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise KernelError("sample: logits must be a row-major float32 matrix")
    n, vocab = logits.shape
    if temperature.dtype != torch.float32 or temperature.numel() != n:
        raise KernelError("sample: temperature must be float32 [n]")
    for t, what in ((seeds, "seeds"), (steps, "steps")):
        if t.dtype != torch.int64 or t.numel() != n or not t.is_contiguous():
            raise KernelError(f"sample: {what} must be int64 [n]")
    if top_k is not None and top_k.numel() != n:
        raise KernelError("sample: top_k must be int32 [n]")
    if out is None:
        out = torch.empty((n,), dtype=torch.int32, device=logits.device)
    elif out.dtype != torch.int32 or tuple(out.shape) != (n,) or not out.is_contiguous() or out.device != logits.device:
        raise KernelError("sample: out must be int32 [n] beside the logits")
    chunks = sample_chunks(n, vocab) if top_k is None and logits.stride(0) % 4 == 0 and logits.data_ptr() % 16 == 0 else 1
    if chunks > 1:
        candidates = torch.empty((n, chunks, 2), dtype=torch.int32, device=logits.device)
        check(
            core().tl_sample_chunks(
                logits.data_ptr(), logits.stride(0), n, vocab, temperature.data_ptr(), seeds.data_ptr(), steps.data_ptr(),
                chunks, candidates.data_ptr(), out.data_ptr(), _stream(),
            )
        )
        return out
    check(
        core().tl_sample(
            logits.data_ptr(), logits.stride(0), n, vocab, temperature.data_ptr(), _ptr(top_k),
            seeds.data_ptr(), steps.data_ptr(), out.data_ptr(), _stream(),
        )
    )
    return out


def sample_chunks(n_rows: int, vocab: int) -> int:
    """Blocks per row for ``sample``: one block does a row of 128k logits in 11 us (argmax) to 70 us
    (temperature), on one of 256 CUs; with few rows the row is cut so that about 256 blocks work,
    no piece shorter than 8,192 logits (the second kernel that picks among the pieces costs a few
    microseconds, which a short row does not win back)."""
    return max(1, min(256 // max(n_rows, 1), vocab // 8192, 16))


def philox_uniform(seed: int, step: int, n: int, device) -> torch.Tensor:
    """The uniforms the sampler draws for (seed, step) at indices 0..n-1."""
    out = torch.empty((n,), dtype=torch.float32, device=device)
    check(core().tl_philox_uniform(seed & (2**64 - 1), step & (2**64 - 1), out.data_ptr(), n, _stream()))
    return out
