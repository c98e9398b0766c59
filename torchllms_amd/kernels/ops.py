"""The kernels as functions of ``torch`` tensors.

Every function checks on the host that shapes, dtypes and devices are what the kernel and its grid
assume, launches on torch's current HIP stream and raises ``KernelError`` when a launcher refuses.
Tensors must live on the GPU: there is no CPU path.
"""

from __future__ import annotations

from typing import Optional

import torch

from .lib import KernelError, check, core, variant

F32, BF16 = 0, 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise KernelError(f"unsupported dtype {dtype}; kernels take float32 and bfloat16") from None


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _gpu(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("kernel arguments must be GPU tensors (there is no CPU path)")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _i32(t: Optional[torch.Tensor], what: str) -> None:
    if t is not None and (t.dtype != torch.int32 or not t.is_contiguous()):
        raise KernelError(f"{what} must be a contiguous int32 tensor")


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


def attention_generic(
    qkv: torch.Tensor,
    n_q_heads: int,
    n_kv_heads: int,
    head_dim: int,
    k_pages: torch.Tensor,
    v_pages: torch.Tensor,
    token_seq: torch.Tensor,
    positions: torch.Tensor,
    block_table: torch.Tensor,
    window: int,
    scale: float,
    out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Attention of each token's query heads (the first Hq * dh columns of ``qkv``) over the paged
    keys and values of its request; returns [n, Hq * dh]."""
    _gpu(qkv, k_pages, v_pages, token_seq, positions, block_table)
    _i32(token_seq, "token_seq")
    _i32(positions, "positions")
    n = qkv.shape[0]
    if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] < n_q_heads * head_dim:
        raise KernelError("attention: qkv must be row-major with at least Hq * dh columns")
    if token_seq.numel() != n or positions.numel() != n:
        raise KernelError("attention: token_seq and positions need one entry per token")
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or block_table.stride(1) != 1:
        raise KernelError("attention: block_table must be an int32 matrix")
    page_size = k_pages.shape[2]
    for pg in (k_pages, v_pages):
        if pg.dim() != 4 or pg.shape[1:] != (n_kv_heads, page_size, head_dim) or pg.dtype != qkv.dtype or not pg.is_contiguous():
            raise KernelError("attention: pages must be contiguous [pages, Hkv, page_size, dh] of the query's dtype")
    if out is None:
        out = torch.empty((n, n_q_heads * head_dim), dtype=qkv.dtype, device=qkv.device)
    check(
        core().tl_attention_generic(
            qkv.data_ptr(), qkv.stride(0), out.data_ptr(), out.stride(0), k_pages.data_ptr(), v_pages.data_ptr(),
            token_seq.data_ptr(), positions.data_ptr(), block_table.data_ptr(), block_table.stride(0), n,
            n_q_heads, n_kv_heads, head_dim, page_size, window, float(scale), dtype_code(qkv.dtype), _stream(),
        )
    )
    return out


def gemm_f32(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``x @ w.T`` in true 32-bit arithmetic; x [m, k], w [n, k], both float32."""
    _gpu(x, w)
    if x.dtype != torch.float32 or w.dtype != torch.float32:
        raise KernelError("gemm_f32 takes float32 tensors")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or x.stride(1) != 1 or w.stride(1) != 1:
        raise KernelError(f"gemm_f32: shapes {tuple(x.shape)} x {tuple(w.shape)}^T do not match")
    m, k = x.shape
    n = w.shape[0]
    out = torch.empty((m, n), dtype=torch.float32, device=x.device)
    check(core().tl_gemm_f32(x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0), m, n, k, _stream()))
    return out


STREAM_MAX_ROWS = 16  # what the weight-streaming kernel takes
#: shapes that were never measured (see ``tune_linear``) use the weight-streaming kernel up to this
#: many elements: small matrices are where the library's launch and tail costs weigh most
STREAM_MAX_ELEMENTS = 1 << 28


def gemm_stream(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16, waves: int = 0) -> torch.Tensor:
    """``x @ w.T`` for at most 16 rows of bfloat16 ``x`` with the kernel that fetches W coalesced
    and transposes it through LDS; the result is bfloat16 or float32."""
    _gpu(x, w)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("gemm_stream takes bfloat16 tensors")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or x.stride(1) != 1 or w.stride(1) != 1:
        raise KernelError(f"gemm_stream: shapes {tuple(x.shape)} x {tuple(w.shape)}^T do not match")
    m, k = x.shape
    n = w.shape[0]
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    check(
        core().tl_gemm_stream(
            x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0), m, n, k,
            dtype_code(out_dtype), waves, _stream(),
        )
    )
    return out


WIDE_MAX_ROWS = 128


def _wide_shapes(x: torch.Tensor, w: torch.Tensor, what: str) -> None:
    _gpu(x, w)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError(f"{what} takes bfloat16 tensors")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or x.stride(1) != 1 or w.stride(1) != 1:
        raise KernelError(f"{what}: shapes {tuple(x.shape)} x {tuple(w.shape)}^T do not match")


class SplitSums:
    """A matrix product that was split along K and not yet added up: ``partial`` float32
    [splits, rows, columns].  The product is the sum of the slices in their order, rounded to
    ``dtype``; ``rmsnorm`` takes it as ``delta`` and adds the slices while it reads them, which
    saves the kernel that would otherwise do nothing else."""

    def __init__(self, partial: torch.Tensor, dtype: torch.dtype):
        self.partial = partial
        self.dtype = dtype

    @property
    def shape(self):
        return tuple(self.partial.shape[1:])

    def resolve(self) -> torch.Tensor:
        splits, m, n = self.partial.shape
        out = torch.empty((m, n), dtype=self.dtype, device=self.partial.device)
        check(core().tl_gemm_wide_reduce(self.partial.data_ptr(), out.data_ptr(), out.stride(0), m, n, splits, dtype_code(self.dtype), _stream()))
        return out


def resolved(x):
    """``x`` as a tensor: a ``SplitSums`` is added up, a tensor is returned as it is.  For code that
    does arithmetic of its own on what a mixer or feed-forward returned."""
    return x.resolve() if isinstance(x, SplitSums) else x


def gemm_wide(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16, strips_per_wave: int = 1,
              k_splits: int = 1, stages: int = 3, leave_split: bool = False):
    """``x @ w.T`` for at most 128 rows of bfloat16 ``x`` (K a multiple of 128) with the kernel whose
    blocks share their slice of ``x`` through LDS; ``k_splits`` > 1 cuts K over several blocks whose
    32-bit partial sums a second kernel adds, or, with ``leave_split``, come back as ``SplitSums``."""
    _wide_shapes(x, w, "gemm_wide")
    m, k = x.shape
    n = w.shape[0]
    if leave_split:
        if n % 4:
            raise KernelError("gemm_wide: split sums need a number of columns that is a multiple of 4")
        used = core().tl_gemm_wide_splits(k, k_splits)
        partial = torch.empty((max(used, 1), m, n), dtype=torch.float32, device=x.device)
        check(
            core().tl_gemm_wide(
                x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), None, n, m, n, k,
                dtype_code(out_dtype), strips_per_wave, k_splits, stages, 0, partial.data_ptr(), _stream(),
            )
        )
        return SplitSums(partial, out_dtype)
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    partial = torch.empty((k_splits, m, n), dtype=torch.float32, device=x.device) if k_splits > 1 else None
    check(
        core().tl_gemm_wide(
            x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0), m, n, k,
            dtype_code(out_dtype), strips_per_wave, k_splits, stages, 1, _ptr(partial), _stream(),
        )
    )
    return out


def gemm_wide_glu(x: torch.Tensor, w: torch.Tensor, strips_per_wave: int = 1, stages: int = 3) -> torch.Tensor:
    """``silu(x @ gate.T) * (x @ up.T)`` for at most 128 rows of bfloat16 ``x`` and ``w`` [2F, K] =
    gate rows | up rows, in one pass over ``w``; rounded as ``silu_mul(linear(x, w))``."""
    _wide_shapes(x, w, "gemm_wide_glu")
    if w.shape[0] % 2:
        raise KernelError("gemm_wide_glu: w must hold gate rows and as many up rows")
    m, k = x.shape
    n = w.shape[0] // 2
    out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    check(
        core().tl_gemm_wide_glu(
            x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0), m, n, k,
            strips_per_wave, stages, _stream(),
        )
    )
    return out


def _qkv_shapes(what, x, w, n_q_heads, n_kv_heads, head_dim, rotary_dim, cos_sin, k_pages, v_pages, slot_mapping, page_size) -> int:
    """Checks the arguments that the fused query|key|value products share; returns the output width."""
    _gpu(x, w, cos_sin, k_pages, v_pages, slot_mapping)
    _i32(slot_mapping, "slot_mapping")
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError(f"{what} takes bfloat16 tensors")
    width = (n_q_heads + 2 * n_kv_heads) * head_dim
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or x.stride(1) != 1 or w.stride(1) != 1 or w.shape[0] != width:
        raise KernelError(f"{what}: shapes {tuple(x.shape)} x {tuple(w.shape)}^T do not match {width} output columns")
    m = x.shape[0]
    if rotary_dim > 0 and (cos_sin is None or cos_sin.dtype != torch.float32 or tuple(cos_sin.shape) != (m, rotary_dim // 2, 2) or not cos_sin.is_contiguous()):
        raise KernelError(f"cos_sin must be contiguous float32 [{m}, {rotary_dim // 2}, 2]")
    if k_pages is not None:
        if v_pages is None or slot_mapping is None or slot_mapping.numel() != m:
            raise KernelError("pages need v_pages and one slot per row")
        for pg in (k_pages, v_pages):
            if pg.dim() != 4 or pg.shape[1:] != (n_kv_heads, page_size, head_dim) or pg.dtype != torch.bfloat16 or not pg.is_contiguous():
                raise KernelError(f"pages must be contiguous bfloat16 [pages, {n_kv_heads}, {page_size}, {head_dim}], got {tuple(pg.shape)} {pg.dtype}")
    return width


def gemm_wide_qkv(
    x: torch.Tensor,
    w: torch.Tensor,
    n_q_heads: int,
    n_kv_heads: int,
    head_dim: int,
    rotary_dim: int,
    cos_sin: Optional[torch.Tensor],
    k_pages: Optional[torch.Tensor],
    v_pages: Optional[torch.Tensor],
    slot_mapping: Optional[torch.Tensor],
    page_size: int,
    strips_per_wave: int = 1,
    k_splits: int = 4,
    stages: int = 3,
) -> torch.Tensor:
    """As ``gemm_stream_qkv`` for at most 128 rows: the product split along K, and the kernel that
    adds the splits rotates the heads and writes keys and values into their pages."""
    width = _qkv_shapes("gemm_wide_qkv", x, w, n_q_heads, n_kv_heads, head_dim, rotary_dim, cos_sin, k_pages, v_pages, slot_mapping, page_size)
    m, k = x.shape
    out = torch.empty((m, width), dtype=torch.bfloat16, device=x.device)
    partial = torch.empty((k_splits, m, width), dtype=torch.float32, device=x.device)
    check(
        core().tl_gemm_wide_qkv(
            x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0), m, k,
            n_q_heads, n_kv_heads, head_dim, rotary_dim, _ptr(cos_sin), _ptr(k_pages), _ptr(v_pages),
            _ptr(slot_mapping), page_size, strips_per_wave, k_splits, stages, partial.data_ptr(), _stream(),
        )
    )
    return out


def gemm_stream_glu(x: torch.Tensor, w: torch.Tensor, waves: int = 0, cols: int = 16) -> torch.Tensor:
    """``silu(x @ gate.T) * (x @ up.T)`` for at most 16 rows of bfloat16 ``x`` and ``w`` [2F, K] =
    gate rows | up rows, in one pass over ``w``; rounded as ``silu_mul(linear(x, w))``.  ``cols``: 16
    or 8 columns of the result per block (8: a launch shaped like the plain product's)."""
    _gpu(x, w)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("gemm_stream_glu takes bfloat16 tensors")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or x.stride(1) != 1 or w.stride(1) != 1 or w.shape[0] % 2:
        raise KernelError(f"gemm_stream_glu: shapes {tuple(x.shape)} x {tuple(w.shape)}^T do not match")
    m, k = x.shape
    n = w.shape[0] // 2
    out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    check(
        core().tl_gemm_stream_glu(
            x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0), m, n, k, waves, cols, _stream(),
        )
    )
    return out


def gemm_stream_qkv(
    x: torch.Tensor,
    w: torch.Tensor,
    n_q_heads: int,
    n_kv_heads: int,
    head_dim: int,
    rotary_dim: int,
    cos_sin: Optional[torch.Tensor],
    k_pages: Optional[torch.Tensor],
    v_pages: Optional[torch.Tensor],
    slot_mapping: Optional[torch.Tensor],
    page_size: int,
    waves: int = 0,
) -> torch.Tensor:
    """The fused projection ``x @ w.T`` of at most 16 rows into query | key | value heads with the
    rotation (interleaved pairs, from the ``rope_table`` of the rows' positions) and the cache
    write in the kernel's epilogue.  Returns [n, (Hq + 2 Hkv) * dh] whose query part is rotated;
    the key and value parts are only filled when no pages are given."""
    width = _qkv_shapes("gemm_stream_qkv", x, w, n_q_heads, n_kv_heads, head_dim, rotary_dim, cos_sin, k_pages, v_pages, slot_mapping, page_size)
    m, k = x.shape
    out = torch.empty((m, width), dtype=torch.bfloat16, device=x.device)
    check(
        core().tl_gemm_stream_qkv(
            x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0), m, k,
            n_q_heads, n_kv_heads, head_dim, rotary_dim, _ptr(cos_sin), _ptr(k_pages), _ptr(v_pages),
            _ptr(slot_mapping), page_size, waves, _stream(),
        )
    )
    return out


def stream_supported(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the weight-streaming kernel can take this product at all."""
    return (
        x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.shape[0] <= STREAM_MAX_ROWS and x.shape[1] % 8 == 0
        and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
    )


def wide_supported(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the kernel for 17 to 128 rows can take this product at all."""
    return (
        x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and STREAM_MAX_ROWS < x.shape[0] <= WIDE_MAX_ROWS
        and x.shape[1] % 128 == 0 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
        and w.data_ptr() % 16 == 0
    )


#: measured choice of bfloat16 kernel by (n, k, row bucket, use); filled by ``tune_linear``:
#:   ("stream", waves[, cols])                     the weight-streaming kernel (waves 0 = its own rule;
#:                                                 cols: columns per block of the gated form, 8 or 16)
#:   ("wide", strips_per_wave, k_splits, stages)   the kernel whose blocks share the activations
#:   None                                          the library
#: Shapes never measured follow the size rule below.
_LINEAR_CHOICE: dict = {}
ROW_BUCKETS = (1, 2, 4, 8, 16, 32, 64, 128)
STREAM_WAVE_CHOICES = (0, 4)
#: (strips per wave, splits of K, buffers) that ``tune_linear`` tries from 17 rows on: whole-K
#: launches for matrices with many rows, splits of K for those with few
WIDE_CHOICES = ((1, 1, 3), (2, 1, 3), (2, 1, 2), (1, 4, 3), (1, 8, 3), (2, 8, 3), (2, 8, 2))


def wide_fits(rows: int, strips_per_wave: int, stages: int) -> bool:
    """Whether the buffers of such a launch fit the 160 KB of LDS: a buffer holds 4 KB for every 16
    rows of the row tile (32, 64 or 128) and 16 KB for every strip per wave."""
    tile = 32 if rows <= 32 else 64 if rows <= 64 else 128
    return stages * (tile // 16 * 4 + strips_per_wave * 16) <= 160

#: how a product is used: alone; as the first half of ``linear_glu`` / ``qkv_rope_store``, whose
#: second half (gate, rotation and cache write) some kernels take into themselves; or ("sum",
#: ``linear_to_sum``) as a term of the residual sum, where the norm that follows adds up a split
#: product for nothing
LINEAR_USES = ("plain", "glu", "qkv", "sum")
#: microseconds that a small kernel between large ones costs in a replayed decode step (measured as
#: the difference between graphs with and without it: 2.7 to 3.1 for a norm of 1 to 64 rows; a kernel
#: trace shows 4.6 and more for every dispatch, an empty one included, which is the profiler's own);
#: ``tune_linear`` charges it to a candidate that leaves the second half of a fused use to a kernel
#: of its own
_TAIL_KERNEL_US = 2.8


def _row_bucket(m: int) -> int:
    for b in ROW_BUCKETS:
        if m <= b:
            return b
    return ROW_BUCKETS[-1]


def _fuses_tail(choice, use: str) -> bool:
    """Whether the kernel of ``choice`` does the second half of ``use`` itself."""
    if use in ("plain", "sum") or choice is None:
        return use in ("plain", "sum")
    if choice[0] == "stream":
        return True
    return choice[2] == 1 if use == "glu" else choice[2] > 1  # the gate ends a whole product, the rotation a split one


def linear_choice(x: torch.Tensor, w: torch.Tensor, use: str = "plain"):
    """Which bfloat16 kernel runs ``x @ w.T``: a tuple as in the table above, or None for the library."""
    m = x.shape[0]
    if m <= STREAM_MAX_ROWS:
        if not stream_supported(x, w):
            return None
        key = (w.shape[0], w.shape[1], _row_bucket(m), use)
        if key in _LINEAR_CHOICE:
            return _LINEAR_CHOICE[key]
        return ("stream", 0) if w.shape[0] * w.shape[1] <= STREAM_MAX_ELEMENTS else None
    if not wide_supported(x, w):
        return None
    return _LINEAR_CHOICE.get((w.shape[0], w.shape[1], _row_bucket(m), use))


_TUNE_FLUSH_BYTES = 512 << 20  # twice the 256 MB of last-level cache


# In inference mode like the engine's steps: torch keeps the random generator's capture state in
# tensors that live as long as any graph does and are updated in place at every capture; were they
# made by a step's capture (inference tensors), a later capture outside inference mode would be
# refused, so every capture of this package runs inside it.
@torch.inference_mode()
def tune_linear(weights, out_dtype: torch.dtype = torch.bfloat16, use: str = "plain", iters: int = 8, report=None) -> None:
    """Measure, for matrices of one shape and every row bucket, which bfloat16 kernel and launch is
    fastest on this GPU, and remember it.  ``weights``: the model's tensors of that shape; ``use``:
    one of ``LINEAR_USES``.  "glu" times the whole gated product as ``linear_glu`` would run it,
    "sum" a product that may stay split; for "qkv" the plain product is timed and a candidate that
    cannot take rotation and cache write into itself is charged the kernel that has to follow it.

    Timing is made like a decode step: the launches are recorded into a HIP graph and replayed (a
    product that needs two kernels is then charged what a second graph node costs, not what a
    second launch from Python costs), they rotate over the tensors, and the caches are flushed
    before every replay, so that the matrices come from HBM as they do in a step.  Shapes already
    measured are left alone, so every engine of a process makes the same choice.  ``report``, if
    given, is called with (row bucket, candidate, microseconds per product) for everything timed."""
    import gc

    weights = [w for w in weights if w.is_cuda and w.dtype == torch.bfloat16 and w.dim() == 2]
    if not weights:
        return
    n, k = weights[0].shape
    if k % 8 or weights[0].stride(0) % 8:
        return
    if use not in LINEAR_USES:
        raise ValueError(f"use must be one of {LINEAR_USES}, got {use!r}")
    if use == "glu" and n % 2:
        raise ValueError(f"a gated matrix holds gate rows and as many up rows, got {n} rows")
    if all((n, k, bucket, use) in _LINEAR_CHOICE for bucket in ROW_BUCKETS):
        return
    device = weights[0].device
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    # read, not written, before every replay: written lines would still be on their way to HBM
    # while the products are timed
    flush = torch.zeros(_TUNE_FLUSH_BYTES // 4, dtype=torch.float32, device=device)  # (summed without a conversion pass)

    def clock(fn) -> float:
        for i in range(2):  # loads the kernel's code and lets it ask for its LDS before the recording
            fn(weights[i % len(weights)])
        torch.cuda.synchronize(device)
        graph = torch.cuda.CUDAGraph()
        # nothing may be destroyed while the stream is recording: the collector stays off meanwhile
        collecting = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(graph):
                for i in range(iters):
                    fn(weights[(i + 2) % len(weights)])
        finally:
            if collecting:
                gc.enable()
        best = float("inf")
        for _ in range(3):  # the least of three replays: a stall of the machine does not decide
            flush.sum()
            start.record()
            graph.replay()
            stop.record()
            stop.synchronize()
            best = min(best, start.elapsed_time(stop))
        return best

    def cost(bucket, choice, fn) -> float:
        tail = _TAIL_KERNEL_US * 1e-3 * iters if use == "qkv" and not _fuses_tail(choice, use) else 0.0
        t = clock(fn) + tail
        if report is not None:
            report(bucket, choice, t / iters * 1e3)
        return t

    for bucket in ROW_BUCKETS:
        if (n, k, bucket, use) in _LINEAR_CHOICE:
            continue
        x = torch.randn((bucket, k), device=device, dtype=torch.float32).to(torch.bfloat16)

        def run(choice):
            if use == "glu":
                return lambda w: _run_glu(choice, x, w)
            return lambda w: _run_choice(choice, x, w, out_dtype, leave_split=use == "sum")

        best, best_time = None, cost(bucket, None, run(None))
        if bucket <= STREAM_MAX_ROWS and use == "glu":
            candidates = [("stream", waves, cols) for waves in STREAM_WAVE_CHOICES for cols in (8, 16)]
        elif bucket <= STREAM_MAX_ROWS:
            candidates = [("stream", waves) for waves in STREAM_WAVE_CHOICES]
        elif wide_supported(x, weights[0]):
            candidates = [("wide",) + c for c in WIDE_CHOICES if c[1] <= k // 128 and wide_fits(bucket, c[0], c[2])]
            # (two buffers are only tried where three do not fit)
            candidates = [c for c in candidates if c[3] == 3 or not wide_fits(bucket, c[1], 3)]
        else:
            candidates = []
        for choice in candidates:
            t = cost(bucket, choice, run(choice))
            if t < best_time:
                best, best_time = choice, t
        _LINEAR_CHOICE[(n, k, bucket, use)] = best


def _run_choice(choice, x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, leave_split: bool = False):
    if choice is None:
        y = torch.nn.functional.linear(x, w)
        return y if y.dtype == out_dtype else y.to(out_dtype)
    if choice[0] == "stream":
        return gemm_stream(x, w, out_dtype, choice[1])
    leave_split = leave_split and choice[2] > 1 and w.shape[0] % 4 == 0
    return gemm_wide(x, w, out_dtype, choice[1], choice[2], choice[3], leave_split)


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``x @ w.T``.  float32: the true 32-bit kernel.  bfloat16: for up to 128 rows (decode steps)
    one of the two MFMA kernels that are built around reading ``w`` once, or the BLAS library's
    matrix product, whichever was measured faster for the shape (``tune_linear``); for more rows the
    library, as the reference uses its library's (torchllms/models/networks.py:474-493).
    ``out_dtype`` float32 asks for 32-bit results from bfloat16 inputs (logits)."""
    if x.dtype == torch.float32:
        return gemm_f32(x, w)
    _gpu(x, w)
    out_dtype = out_dtype or x.dtype
    return _run_choice(linear_choice(x, w), x, w, out_dtype)


def linear_to_sum(x: torch.Tensor, w: torch.Tensor):
    """``x @ w.T`` for a result that is only ever added to the residual stream by ``rmsnorm(...,
    delta=...)``: a tensor, or ``SplitSums`` when the product was split along K, which that
    ``rmsnorm`` adds up while it reads them."""
    if x.dtype == torch.float32:
        return gemm_f32(x, w)
    _gpu(x, w)
    return _run_choice(linear_choice(x, w, "sum"), x, w, x.dtype, leave_split=True)


def linear_glu(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``silu(x @ gate.T) * (x @ up.T)`` for ``w`` [2F, K] = gate rows | up rows: one fused kernel
    where one of the decode kernels serves the shape, else the product followed by the gate."""
    if x.dtype != torch.bfloat16:
        return silu_mul(linear(x, w))
    _gpu(x, w)
    return _run_glu(linear_choice(x, w, "glu"), x, w)


def _run_glu(choice, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    if choice is not None and choice[0] == "stream":
        return gemm_stream_glu(x, w, choice[1], choice[2] if len(choice) > 2 else 16)
    if choice is not None and choice[0] == "wide" and choice[2] == 1:
        return gemm_wide_glu(x, w, choice[1], choice[3])
    return silu_mul(_run_choice(choice, x, w, x.dtype))


def qkv_rope_store(
    x: torch.Tensor,
    w: torch.Tensor,
    bias: Optional[torch.Tensor],
    n_q_heads: int,
    n_kv_heads: int,
    head_dim: int,
    positions: torch.Tensor,
    inv_freq: Optional[torch.Tensor],
    rotary_dim: int,
    pairing: int,
    cos_sin: Optional[torch.Tensor],
    k_pages: Optional[torch.Tensor],
    v_pages: Optional[torch.Tensor],
    slot_mapping: Optional[torch.Tensor],
    page_size: int,
) -> torch.Tensor:
    """Projection into query | key | value heads, rotation of queries and keys by position, keys
    and values appended to their pages; returns the row-major [n, (Hq + 2 Hkv) * dh] buffer whose
    query part the attention kernels read.  Fused into the product's own kernels where one of the
    decode kernels serves it (at most 128 bfloat16 rows, no bias, interleaved pairs, head size a
    multiple of 4), else product, bias and rotary kernels in turn."""
    if x.dtype == torch.bfloat16:
        _gpu(x, w)
        choice = linear_choice(x, w, "qkv")
        fusable = bias is None and head_dim % 4 == 0 and (rotary_dim == 0 or (pairing == 0 and cos_sin is not None))
        if fusable and choice is not None and choice[0] == "stream":
            return gemm_stream_qkv(
                x, w, n_q_heads, n_kv_heads, head_dim, rotary_dim, cos_sin, k_pages, v_pages, slot_mapping, page_size, choice[1]
            )
        # (a product that is not split ends without a second kernel, so the rotary kernel follows it)
        if fusable and choice is not None and choice[0] == "wide" and choice[2] > 1:
            return gemm_wide_qkv(
                x, w, n_q_heads, n_kv_heads, head_dim, rotary_dim, cos_sin, k_pages, v_pages, slot_mapping, page_size,
                choice[1], choice[2], choice[3],
            )
        qkv = _run_choice(choice, x, w, x.dtype)
    else:
        qkv = linear(x, w)
    if bias is not None:
        add_bias_(qkv, bias)
    rope_kv_write(
        qkv, n_q_heads, n_kv_heads, head_dim, positions, inv_freq, rotary_dim, pairing, k_pages, v_pages,
        slot_mapping, page_size, cos_sin=cos_sin,
    )
    return qkv


def sample(
    logits: torch.Tensor,
    temperature: torch.Tensor,
    seeds: torch.Tensor,
    steps: torch.Tensor,
    top_k: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """One token per row of float32 ``logits`` [n, vocab]; see csrc/sampling.hip for the rule.  Without
    top-k and with few rows, several blocks share a row (``sample_chunks``); the tokens are the same.
    ``temperature`` float32 [n]; ``seeds``/``steps`` int64 [n] (read as unsigned); ``top_k`` int32 [n]."""
    _gpu(logits, temperature, seeds, steps, top_k)
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
    out = torch.empty((n,), dtype=torch.int32, device=logits.device)
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


# ----------------------------------------------------------------------------- decode attention (bfloat16, MFMA)
_P, _I, _F = __import__("ctypes").c_void_p, __import__("ctypes").c_int, __import__("ctypes").c_float
_DECODE_SIGNATURES = {
    "tl_attn_decode": [_P, _I, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _I, _I, _P, _P, _P],
}
DECODE_HEAD_DIMS = (32, 64, 128, 256)
_DECODE_BLOCK_KEYS = 64  # keys one block pass covers (4 waves x 16): splits are multiples of it


def decode_attention_supported(dtype: torch.dtype, n_q_heads: int, n_kv_heads: int, head_dim: int) -> bool:
    """Whether the MFMA decode kernel takes these sizes (else the plain kernel runs)."""
    if dtype != torch.bfloat16 or head_dim not in DECODE_HEAD_DIMS or n_q_heads % n_kv_heads:
        return False
    return n_q_heads // n_kv_heads <= (16 if head_dim <= 128 else 8)


_DECODE_MIN_SPLIT = 256  # keys: shorter splits cost more in launch and merge than they gain in spread


_DECODE_UNEVEN_SPLIT = 1024  # keys: the longest split when requests differ much in length


def plan_decode_splits(n_tokens: int, n_kv_heads: int, longest: int, target_blocks: int = 512, uneven: bool = False):
    """``(split_size, n_splits)`` for a decode launch whose longest visible key range (counted from
    its 16-aligned start) is ``longest``: enough splits for about two blocks on each of the 256
    CUs, none shorter than 256 keys.  Measured from one request of 131,072 tokens to 128 requests
    of 2,048, 512 blocks were the best or within 2% of it: a block's waves keep enough loads in
    flight by themselves, and every further split costs its start, its partial results and its
    share of the merge.  A batch with 512 (request, kv head) pairs or more is not split at all,
    if the requests are about equally long.  (Alone and on pages in random order, 8 requests of
    8,192 tokens ran a little faster with four splits of 2,048 keys than with eight of 1,024; inside
    the decode step it was the other way round, 52.9 against 49.5 us, and the step decides.)

    ``uneven``: the requests differ much in length.  Then all blocks of such a launch would be
    resident at once and stay where they were put, a CU with long requests' blocks working on
    when its neighbours have finished; with splits of at most 1,024 keys there are several times
    more blocks than fit, and those that wait go where others end.  (64 requests of 128 to 4,608
    tokens: 30% less time than unsplit; 64 equal ones: 10% more, hence the switch.)"""
    pairs = max(n_tokens * n_kv_heads, 1)
    want = max(-(-target_blocks // pairs), 1)
    split = -(-max(longest, 1) // want)
    if uneven:
        split = min(split, _DECODE_UNEVEN_SPLIT)
    split = max(-(-split // _DECODE_BLOCK_KEYS) * _DECODE_BLOCK_KEYS, _DECODE_MIN_SPLIT)
    # splits of 256 keys only while 512 keys would leave fewer than one block for each CU (measured
    # with cold caches: 2 requests of 8,192 tokens 23.4 against 25.8 us, 8 of 2,048 21.7 against 23.3,
    # 2 of 4,096, where 512 keys give 128 blocks, 20.0 against 18.4)
    if split < 2 * _DECODE_MIN_SPLIT and pairs * -(-max(longest, 1) // (2 * _DECODE_MIN_SPLIT)) >= 256:
        split = 2 * _DECODE_MIN_SPLIT
    return split, max(-(-max(longest, 1) // split), 1)


def attention_decode(
    qkv: torch.Tensor,
    n_q_heads: int,
    n_kv_heads: int,
    head_dim: int,
    k_pages: torch.Tensor,
    v_pages: torch.Tensor,
    token_seq: torch.Tensor,
    positions: torch.Tensor,
    block_table: torch.Tensor,
    window: int,
    scale: float,
    longest: int,
    out: Optional[torch.Tensor] = None,
    split_size: Optional[int] = None,
    uneven: bool = False,
) -> torch.Tensor:
    """Attention of single-token queries over their requests' pages with the split-KV MFMA kernel.
    ``longest``: an upper bound of any token's visible key range, counted from its 16-aligned first
    visible key (position + 1 without a window)."""
    _gpu(qkv, k_pages, v_pages, token_seq, positions, block_table)
    _i32(token_seq, "token_seq")
    _i32(positions, "positions")
    if qkv.dtype != torch.bfloat16:
        raise KernelError("attention_decode takes bfloat16")
    n = token_seq.numel()
    if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[0] < n or qkv.shape[1] < n_q_heads * head_dim:
        raise KernelError("attention_decode: qkv must be row-major with a row per token and at least Hq * dh columns")
    if positions.numel() != n:
        raise KernelError("attention_decode: one position per token")
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or block_table.stride(1) != 1:
        raise KernelError("attention_decode: block_table must be an int32 matrix")
    page_size = k_pages.shape[2]
    for pg in (k_pages, v_pages):
        if pg.dim() != 4 or pg.shape[1:] != (n_kv_heads, page_size, head_dim) or pg.dtype != qkv.dtype or not pg.is_contiguous():
            raise KernelError("attention_decode: pages must be contiguous [pages, Hkv, page_size, dh] bfloat16")
    if out is None:
        out = torch.empty((n, n_q_heads * head_dim), dtype=qkv.dtype, device=qkv.device)
    if split_size is None:
        split_size, n_splits = plan_decode_splits(n, n_kv_heads, longest, uneven=uneven)
    else:
        n_splits = max(-(-max(longest, 1) // split_size), 1)
    ws_o = ws_ml = None
    if n_splits > 1:
        ws_o = torch.empty((n * n_q_heads * n_splits * head_dim,), dtype=torch.float32, device=qkv.device)
        ws_ml = torch.empty((n * n_q_heads * n_splits * 2,), dtype=torch.float32, device=qkv.device)
    lib = variant("attn_decode", head_dim, _DECODE_SIGNATURES)
    check(
        lib.tl_attn_decode(
            qkv.data_ptr(), qkv.stride(0), out.data_ptr(), out.stride(0), k_pages.data_ptr(), v_pages.data_ptr(),
            token_seq.data_ptr(), positions.data_ptr(), block_table.data_ptr(), block_table.stride(0), n,
            n_q_heads, n_kv_heads, head_dim, page_size, window, float(scale), split_size, n_splits,
            _ptr(ws_o), _ptr(ws_ml), _stream(),
        ),
        lib,
        "tl_variant_last_error",
    )
    return out


# ----------------------------------------------------------------------------- prefill attention (bfloat16, MFMA)
_PREFILL_SIGNATURES = {
    "tl_attn_prefill": [_P, _I, _P, _I, _P, _P, _P, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P],
}
PREFILL_HEAD_DIMS = (32, 64, 128, 256)


def prefill_attention_supported(dtype: torch.dtype, n_q_heads: int, n_kv_heads: int, head_dim: int) -> bool:
    """Whether the MFMA prefill kernel takes these sizes (else the plain kernel runs)."""
    return dtype == torch.bfloat16 and head_dim in PREFILL_HEAD_DIMS and n_q_heads % n_kv_heads == 0 and n_q_heads // n_kv_heads <= 16


def prefill_queries_per_tile(n_q_heads: int, n_kv_heads: int, head_dim: int) -> int:
    """Queries one block of the prefill kernel covers: its MFMA columns (128, or 64 at head size 256)
    divided by the group size rounded up to a power of two."""
    group = n_q_heads // n_kv_heads
    rp = 1
    while rp < group:
        rp *= 2
    return (128 if head_dim <= 128 else 64) // rp


#: blocks of the prefill kernel that the GPU holds at once: 256 CUs, two blocks each
PREFILL_RESIDENT_BLOCKS = 512
#: launches of up to this many blocks run with two sets of waves per block (measured at head size
#: 128: 512 blocks 87 -> 72 us, 1,024 blocks even, 2,048 blocks 800 -> 890 us)
PREFILL_SPLIT_BLOCKS = 768


def prefill_key_groups(n_tiles: int, n_kv_heads: int) -> int:
    """Sets of waves per block of the prefill kernel.  A launch whose blocks all fit the GPU at once
    takes as long as its longest block; with two sets of waves, each with every second tile of keys,
    that block's chain is half as long.  A launch of many more blocks keeps the CUs busy anyway, and
    there two independent blocks on a CU overlap better than two sets of waves in step."""
    return 2 if n_tiles * n_kv_heads <= PREFILL_SPLIT_BLOCKS else 1


def prefill_tile_count(qo_indptr, first_row: int, n_rows: int, queries_per_tile: int) -> int:
    return sum(-(-(int(qo_indptr[r + 1]) - int(qo_indptr[r])) // queries_per_tile) for r in range(first_row, n_rows))


def prefill_tiles(qo_indptr, first_row: int, n_rows: int, queries_per_tile: int, kv_lens=None, window: int = 0,
                  n_kv_heads: int = 1, key_groups: int = 1):
    """Host lists ``(tile_row, tile_q0)`` that cut rows ``first_row .. n_rows-1`` into query tiles.

    With ``kv_lens`` the tiles are put in the order that balances the launch: a tile's cost is the
    number of keys it sees, and late tiles of a causal prompt see many times more than early ones.
    Blocks are handed to the CUs in launch order.  When there are far more blocks than fit at once,
    longest first lets short ones fill the gaps at the end; when about all fit at once, the first
    half of the launch takes the long tiles in descending order and the second half the short ones in
    ascending order, so that the blocks that meet on a CU have complementary lengths.  With two sets
    of waves a block (``key_groups`` = 2) a CU holds one block at a time: longest first."""
    rows, q0s, costs = [], [], []
    for r in range(first_row, n_rows):
        q_len = int(qo_indptr[r + 1]) - int(qo_indptr[r])
        pos0 = (int(kv_lens[r]) - q_len) if kv_lens is not None else 0
        for q0 in range(0, q_len, queries_per_tile):
            rows.append(r)
            q0s.append(q0)
            hi = pos0 + min(q0 + queries_per_tile, q_len) - 1
            lo = max(pos0 + q0 - window + 1, 0) if window > 0 else 0
            costs.append(hi - lo + 1)
    if kv_lens is None or len(rows) < 2:
        return rows, q0s
    order = sorted(range(len(rows)), key=lambda i: -costs[i])
    if key_groups == 1 and len(rows) * n_kv_heads <= 2 * PREFILL_RESIDENT_BLOCKS:
        half = (len(order) + 1) // 2
        order = order[:half] + order[half:][::-1]
    return [rows[i] for i in order], [q0s[i] for i in order]


def attention_prefill(
    qkv: torch.Tensor,
    n_q_heads: int,
    n_kv_heads: int,
    head_dim: int,
    k_pages: torch.Tensor,
    v_pages: torch.Tensor,
    qo_indptr: torch.Tensor,
    kv_lens: torch.Tensor,
    block_table: torch.Tensor,
    tile_row: torch.Tensor,
    tile_q0: torch.Tensor,
    window: int,
    scale: float,
    out: torch.Tensor,
    key_groups: int = 1,
) -> torch.Tensor:
    """Causal attention of the rows named by the tile lists (see ``prefill_tiles``) with the MFMA
    prefill kernel.  Token t of ``qkv`` / ``out`` is token t of ``qo_indptr``'s numbering.
    ``key_groups`` = 2: two sets of waves per block share a tile's keys between them."""
    _gpu(qkv, k_pages, v_pages, qo_indptr, kv_lens, block_table, tile_row, tile_q0, out)
    for t, what in ((qo_indptr, "qo_indptr"), (kv_lens, "kv_lens"), (tile_row, "tile_row"), (tile_q0, "tile_q0")):
        _i32(t, what)
    if qkv.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise KernelError("attention_prefill takes bfloat16")
    if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] < n_q_heads * head_dim:
        raise KernelError("attention_prefill: qkv must be row-major with at least Hq * dh columns")
    if out.dim() != 2 or out.stride(1) != 1 or out.shape[0] != qkv.shape[0] or out.shape[1] < n_q_heads * head_dim:
        raise KernelError("attention_prefill: out must be row-major [tokens, >= Hq * dh]")
    if tile_row.numel() != tile_q0.numel():
        raise KernelError("attention_prefill: tile lists differ in length")
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or block_table.stride(1) != 1:
        raise KernelError("attention_prefill: block_table must be an int32 matrix")
    if kv_lens.numel() != block_table.shape[0] or qo_indptr.numel() != kv_lens.numel() + 1:
        raise KernelError("attention_prefill: qo_indptr, kv_lens and block_table disagree about the rows")
    page_size = k_pages.shape[2]
    for pg in (k_pages, v_pages):
        if pg.dim() != 4 or pg.shape[1:] != (n_kv_heads, page_size, head_dim) or pg.dtype != qkv.dtype or not pg.is_contiguous():
            raise KernelError("attention_prefill: pages must be contiguous [pages, Hkv, page_size, dh] bfloat16")
    lib = variant("attn_prefill", head_dim, _PREFILL_SIGNATURES)
    check(
        lib.tl_attn_prefill(
            qkv.data_ptr(), qkv.stride(0), out.data_ptr(), out.stride(0), k_pages.data_ptr(), v_pages.data_ptr(),
            qo_indptr.data_ptr(), kv_lens.data_ptr(), block_table.data_ptr(), block_table.stride(0),
            tile_row.data_ptr(), tile_q0.data_ptr(), tile_row.numel(), n_q_heads, n_kv_heads, head_dim, page_size,
            window, float(scale), int(key_groups), _stream(),
        ),
        lib,
        "tl_variant_last_error",
    )
    return out
