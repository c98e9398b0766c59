"""Embedding, RMS norm, rotary position encoding with the cache write, gate and bias: the kernels
that move rows through memory once."""

from __future__ import annotations

from typing import Optional

import torch

from .base import (  # noqa: F401
    BF16,
    F32,
    KernelError,
    SplitSums,
    Unfinished,
    _gpu,
    _i32,
    _ptr,
    _stream,
    check,
    core,
    device_facts,
    dtype_code,
    resolved,
    variant,
)


def rmsnorm_max_hidden() -> int:
    """The widest row the norm kernels take: a row is kept in LDS as 32-bit floats (the device's LDS,
    160 KB on gfx950, less 1 KB)."""
    return (device_facts()[1] - 1024) // 4


def embed(tokens: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """``table[tokens]``; tokens int32 [n], table [vocab, hidden].  The caller has checked ids < vocab."""
    _gpu(tokens, table)
    _i32(tokens, "tokens")
    if table.dim() != 2 or not table.is_contiguous():
        raise KernelError("embedding table must be a contiguous matrix")
    n, hidden = tokens.numel(), table.shape[1]
    out = torch.empty((n, hidden), dtype=table.dtype, device=table.device)
    check(core().tl_embed(tokens.data_ptr(), table.data_ptr(), out.data_ptr(), n, hidden, dtype_code(table.dtype), _stream()))
    return out


def rmsnorm(
    x: torch.Tensor,
    weight: torch.Tensor,
    eps: float,
    delta: Optional[torch.Tensor] = None,
    rows: Optional[torch.Tensor] = None,
    return_sum: bool = False,
):
    """RMS norm of ``x (+ delta)`` row by row, optionally of the rows ``rows`` only.  ``delta`` may be
    a ``SplitSums``: the kernel then adds the splits itself (where it takes the width, else they are
    added first).

    Returns ``y`` or, with ``return_sum``, ``(x + delta, y)``.
    """
    if isinstance(delta, SplitSums):
        hidden = x.shape[-1]
        if x.dtype == torch.bfloat16 and hidden % 8 == 0 and hidden <= 8192 and delta.shape == tuple(x.shape):
            return _rmsnorm_split(x, weight, eps, delta, rows, return_sum)
        delta = delta.resolve()
    elif isinstance(delta, Unfinished):
        delta = delta.resolve()
    _gpu(x, weight, delta, rows)
    _i32(rows, "rows")
    if x.dim() != 2 or not x.is_contiguous():
        raise KernelError("rmsnorm input must be a contiguous [rows, hidden] tensor")
    hidden = x.shape[1]
    if weight.shape != (hidden,) or not weight.is_contiguous():
        raise KernelError(f"rmsnorm weight must have shape ({hidden},), got {tuple(weight.shape)}")
    if delta is not None and (delta.shape != x.shape or delta.dtype != x.dtype or not delta.is_contiguous()):
        raise KernelError("rmsnorm delta must match the input")
    if rows is not None and return_sum:
        raise KernelError("rmsnorm cannot return the sum together with a row gather")
    n = x.shape[0] if rows is None else rows.numel()
    y = torch.empty((n, hidden), dtype=x.dtype, device=x.device)
    h_out = torch.empty_like(x) if return_sum else None
    check(
        core().tl_rmsnorm(
            x.data_ptr(), _ptr(delta), _ptr(rows), weight.data_ptr(), dtype_code(weight.dtype),
            _ptr(h_out), y.data_ptr(), n, hidden, float(eps), dtype_code(x.dtype), _stream(),
        )
    )
    return (h_out, y) if return_sum else y


def _rmsnorm_split(x, weight, eps, delta: "SplitSums", rows, return_sum):
    _gpu(x, weight, rows)
    _i32(rows, "rows")
    if x.dim() != 2 or not x.is_contiguous():
        raise KernelError("rmsnorm input must be a contiguous [rows, hidden] tensor")
    hidden = x.shape[1]
    if weight.shape != (hidden,) or not weight.is_contiguous():
        raise KernelError(f"rmsnorm weight must have shape ({hidden},), got {tuple(weight.shape)}")
    if rows is not None and return_sum:
        raise KernelError("rmsnorm cannot return the sum together with a row gather")
    n = x.shape[0] if rows is None else rows.numel()
    y = torch.empty((n, hidden), dtype=x.dtype, device=x.device)
    h_out = torch.empty_like(x) if return_sum else None
    part = delta.partial
    check(
        core().tl_rmsnorm_split(
            x.data_ptr(), part.data_ptr(), part.shape[0], part.stride(0), _ptr(rows), weight.data_ptr(),
            dtype_code(weight.dtype), _ptr(h_out), y.data_ptr(), n, hidden, float(eps), _stream(),
        )
    )
    return (h_out, y) if return_sum else y


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """float32 [n, len(inv_freq), 2]: cosine and sine of ``float(position) * inv_freq`` (32-bit angle,
    precise functions).  One table serves every layer of a step that rotates alike."""
    _gpu(positions, inv_freq)
    _i32(positions, "positions")
    if inv_freq.dtype != torch.float32 or inv_freq.dim() != 1 or not inv_freq.is_contiguous() or inv_freq.numel() == 0:
        raise KernelError("inv_freq must be a contiguous float32 vector")
    n, half = positions.numel(), inv_freq.numel()
    out = torch.empty((n, half, 2), dtype=torch.float32, device=positions.device)
    check(core().tl_rope_table(positions.data_ptr(), inv_freq.data_ptr(), n, half, out.data_ptr(), _stream()))
    return out


def rope_kv_write(
    qkv: torch.Tensor,
    n_q_heads: int,
    n_kv_heads: int,
    head_dim: int,
    positions: torch.Tensor,
    inv_freq: Optional[torch.Tensor],
    rotary_dim: int,
    pairing: int,
    k_pages: Optional[torch.Tensor] = None,
    v_pages: Optional[torch.Tensor] = None,
    slot_mapping: Optional[torch.Tensor] = None,
    page_size: int = 0,
    cos_sin: Optional[torch.Tensor] = None,
) -> None:
    """Rotate the query and key heads of ``qkv`` [n, (Hq + 2 Hkv) * dh] by position and store keys
    and values into pages [pages, Hkv, page_size, dh] at ``slot_mapping`` (page * page_size + offset).
    ``cos_sin``: the step's ``rope_table`` for these positions, instead of forming the angles here."""
    _gpu(qkv, positions, inv_freq, k_pages, v_pages, slot_mapping, cos_sin)
    if cos_sin is not None and (cos_sin.dtype != torch.float32 or tuple(cos_sin.shape) != (qkv.shape[0], rotary_dim // 2, 2) or not cos_sin.is_contiguous()):
        raise KernelError(f"cos_sin must be contiguous float32 [{qkv.shape[0]}, {rotary_dim // 2}, 2]")
    _i32(positions, "positions")
    _i32(slot_mapping, "slot_mapping")
    n = qkv.shape[0]
    width = (n_q_heads + 2 * n_kv_heads) * head_dim
    if qkv.dim() != 2 or qkv.shape[1] != width or not qkv.is_contiguous():
        raise KernelError(f"qkv must be contiguous [n, {width}], got {tuple(qkv.shape)}")
    if positions.numel() != n:
        raise KernelError("positions must have one entry per token")
    if rotary_dim > 0 and cos_sin is None:
        if inv_freq is None or inv_freq.dtype != torch.float32 or inv_freq.numel() != rotary_dim // 2 or not inv_freq.is_contiguous():
            raise KernelError(f"inv_freq must be float32 with {rotary_dim // 2} entries")
    if k_pages is not None:
        if v_pages is None or slot_mapping is None or slot_mapping.numel() != n:
            raise KernelError("pages need v_pages and one slot per token")
        for pg in (k_pages, v_pages):
            if pg.dim() != 4 or pg.shape[1:] != (n_kv_heads, page_size, head_dim) or pg.dtype != qkv.dtype or not pg.is_contiguous():
                raise KernelError(
                    f"pages must be contiguous [pages, {n_kv_heads}, {page_size}, {head_dim}] of {qkv.dtype}, got {tuple(pg.shape)} {pg.dtype}"
                )
    check(
        core().tl_rope_kv_write(
            qkv.data_ptr(), n, n_q_heads, n_kv_heads, head_dim, positions.data_ptr(), _ptr(inv_freq), _ptr(cos_sin),
            rotary_dim, pairing, _ptr(k_pages), _ptr(v_pages), _ptr(slot_mapping), page_size,
            dtype_code(qkv.dtype), _stream(),
        )
    )


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """``silu(gate) * up`` for ``gate_up`` [n, 2F] = gate | up."""
    _gpu(gate_up)
    if gate_up.dim() != 2 or gate_up.shape[1] % 2 or not gate_up.is_contiguous():
        raise KernelError("silu_mul input must be contiguous [n, 2F]")
    n, inter = gate_up.shape[0], gate_up.shape[1] // 2
    out = torch.empty((n, inter), dtype=gate_up.dtype, device=gate_up.device)
    check(core().tl_silu_mul(gate_up.data_ptr(), out.data_ptr(), n, inter, dtype_code(gate_up.dtype), _stream()))
    return out


def add_bias_(x: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """In place ``x[:, :len(bias)] += bias`` for a row-major matrix ``x``."""
    _gpu(x, bias)
    if x.dim() != 2 or x.stride(1) != 1 or bias.dim() != 1 or bias.numel() > x.shape[1] or bias.dtype != x.dtype:
        raise KernelError("add_bias: x must be a row-major matrix and bias a vector of its dtype")
    check(core().tl_add_bias(x.data_ptr(), bias.data_ptr(), x.shape[0], bias.numel(), x.stride(0), dtype_code(x.dtype), _stream()))
    return x
