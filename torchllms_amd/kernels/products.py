"""Matrix products: the true 32-bit product, the weight-streaming kernel for up to 16 rows, the kernel
that shares the activations through LDS for 17 to 128 rows, the library for the rest, and the
measurement that decides between them per shape, row count and use."""

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
from .elementwise_ops import add_bias_, rmsnorm, rope_kv_write, rope_table, silu_mul  # noqa: F401

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


#: the widest rows whose norm the streaming products take over: their sums of squares come in width / 16 pieces, and
#: 512 are what a block of eight waves asks for ahead of its walk (more would be fetched at its end, with a wait)
NORMED_ROWS_MAX_WIDTH = 8192


class NormedRows(Unfinished):
    """``rmsnorm(rows, weight, eps)`` of at most 16 bfloat16 rows, not yet computed: ``gained`` are the
    rows times ``weight`` and ``sums`` float32 [pieces, 16] are pieces of each row's sum of squares
    (the rows side by side, at most 16), as ``PendingProduct.added_to`` leaves them.  What is left of the norm is one factor per row,
    which ``linear_glu`` and ``qkv_rope_store`` apply to the sums of ``gained @ w.T`` where the
    weight-streaming kernel runs: norm(x) W^T = ((x * weight) W^T) / sqrt(mean(x^2) + eps)."""

    def __init__(self, rows: torch.Tensor, gained: torch.Tensor, sums: torch.Tensor, eps: float, weight: torch.Tensor):
        self.rows = rows
        self.gained = gained
        self.sums = sums
        self.eps = float(eps)
        self.weight = weight

    @property
    def shape(self):
        return tuple(self.rows.shape)

    @property
    def dtype(self):
        return self.rows.dtype

    def resolve(self) -> torch.Tensor:
        return rmsnorm(self.rows, self.weight, self.eps)

    def kernel_args(self):
        sums = self.sums
        if sums.dtype != torch.float32 or sums.dim() != 2 or sums.shape[1] != 16 or not sums.is_contiguous() or self.gained.shape[0] > 16:
            raise KernelError("the sums of squares do not belong to these rows")
        return sums.data_ptr(), sums.shape[0], self.eps


class PendingProduct(Unfinished):
    """``x @ w.T`` for at most 16 bfloat16 rows, to be run by the weight-streaming kernel with ``waves``
    splits of K, and not yet run: whoever adds it to the residual stream calls ``added_to`` and gets
    the sum from the product's own kernel, with what the norm of the sum needs."""

    def __init__(self, x: torch.Tensor, w: torch.Tensor, waves: int):
        self.x = x
        self.w = w
        self.waves = waves

    @property
    def shape(self):
        return (self.x.shape[0], self.w.shape[0])

    @property
    def dtype(self):
        return self.x.dtype

    def resolve(self) -> torch.Tensor:
        return gemm_stream(self.x, self.w, self.x.dtype, self.waves)

    def added_to(self, h: torch.Tensor, weight: torch.Tensor, eps: float):
        """``(h + x @ w.T, NormedRows of it)`` for a norm with gain ``weight``."""
        rows, gained, sums = gemm_stream_residual(self.x, self.w, h, weight, self.waves)
        return rows, NormedRows(rows, gained, sums, eps, weight)


def gemm_stream_residual(x: torch.Tensor, w: torch.Tensor, h: torch.Tensor, gain: torch.Tensor, waves: int = 0):
    """``rows = h + x @ w.T`` for at most 16 bfloat16 rows (the product rounded to bfloat16 before the
    sum, as if it had been stored), ``rows * gain``, and the sums of squares of ``rows`` by blocks of
    16 columns (float32 [ceil(N / 16), 16]: block by block, the rows side by side, of which the first
    ``len(rows)`` are filled)."""
    _gpu(x, w, h, gain)
    if any(t.dtype != torch.bfloat16 for t in (x, w, h, gain)):
        raise KernelError("gemm_stream_residual takes bfloat16 tensors")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or x.stride(1) != 1 or w.stride(1) != 1:
        raise KernelError(f"gemm_stream_residual: shapes {tuple(x.shape)} x {tuple(w.shape)}^T do not match")
    m, k = x.shape
    n = w.shape[0]
    if tuple(h.shape) != (m, n) or h.stride(1) != 1:
        raise KernelError(f"gemm_stream_residual: rows to add to of shape {tuple(h.shape)}, the product has {(m, n)}")
    if tuple(gain.shape) != (n,) or not gain.is_contiguous():
        raise KernelError(f"gemm_stream_residual: a gain of shape {tuple(gain.shape)} for rows of {n} elements")
    out = torch.empty((2, m, n), dtype=torch.bfloat16, device=x.device)  # the rows, and the rows times the gain
    sums = torch.empty(((n + 15) // 16, 16), dtype=torch.float32, device=x.device)
    check(
        core().tl_gemm_stream_residual(
            x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), h.data_ptr(), h.stride(0), gain.data_ptr(),
            out[0].data_ptr(), out[1].data_ptr(), n, sums.data_ptr(), m, n, k, waves, _stream(),
        )
    )
    return out[0], out[1], sums


def _norm_args(norm: Optional[NormedRows], x: torch.Tensor):
    if norm is None:
        return None, 0, 0.0
    if norm.gained is not x:
        raise KernelError("the sums of squares do not belong to these rows")
    return norm.kernel_args()


WIDE_MAX_ROWS = 128


def wide_shapes(x: torch.Tensor, w: torch.Tensor, what: str) -> None:
    _gpu(x, w)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError(f"{what} takes bfloat16 tensors")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or x.stride(1) != 1 or w.stride(1) != 1:
        raise KernelError(f"{what}: shapes {tuple(x.shape)} x {tuple(w.shape)}^T do not match")


def gemm_wide(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16, strips_per_wave: int = 1,
              k_splits: int = 1, stages: int = 3, leave_split: bool = False):
    """``x @ w.T`` for at most 128 rows of bfloat16 ``x`` (K a multiple of 128) with the kernel whose
    blocks share their slice of ``x`` through LDS; ``k_splits`` > 1 cuts K over several blocks whose
    32-bit partial sums a second kernel adds, or, with ``leave_split``, come back as ``SplitSums``."""
    wide_shapes(x, w, "gemm_wide")
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
    wide_shapes(x, w, "gemm_wide_glu")
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


def qkv_shapes(what, x, w, n_q_heads, n_kv_heads, head_dim, rotary_dim, cos_sin, k_pages, v_pages, slot_mapping, page_size) -> int:
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
    width = qkv_shapes("gemm_wide_qkv", x, w, n_q_heads, n_kv_heads, head_dim, rotary_dim, cos_sin, k_pages, v_pages, slot_mapping, page_size)
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


def gemm_stream_glu(x: torch.Tensor, w: torch.Tensor, waves: int = 0, cols: int = 16, norm: Optional[NormedRows] = None) -> torch.Tensor:
    """``silu(x @ gate.T) * (x @ up.T)`` for at most 16 rows of bfloat16 ``x`` and ``w`` [2F, K] =
    gate rows | up rows, in one pass over ``w``; rounded as ``silu_mul(linear(x, w))``.  ``cols``: 16
    or 8 columns of the result per block (8: a launch shaped like the plain product's).  ``norm``:
    ``NormedRows`` whose ``gained`` rows ``x`` is; the result is then that of the normed rows."""
    _gpu(x, w)
    sums, n_sums, eps = _norm_args(norm, x)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("gemm_stream_glu takes bfloat16 tensors")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or x.stride(1) != 1 or w.stride(1) != 1 or w.shape[0] % 2:
        raise KernelError(f"gemm_stream_glu: shapes {tuple(x.shape)} x {tuple(w.shape)}^T do not match")
    m, k = x.shape
    n = w.shape[0] // 2
    out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    check(
        core().tl_gemm_stream_glu(
            x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0), m, n, k, waves, cols, sums, n_sums, eps,
            _stream(),
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
    norm: Optional[NormedRows] = None,
) -> torch.Tensor:
    """The fused projection ``x @ w.T`` of at most 16 rows into query | key | value heads with the
    rotation (interleaved pairs, from the ``rope_table`` of the rows' positions) and the cache
    write in the kernel's epilogue.  Returns [n, (Hq + 2 Hkv) * dh] whose query part is rotated;
    the key and value parts are only filled when no pages are given.  ``norm``: ``NormedRows`` whose
    ``gained`` rows ``x`` is; the result is then that of the normed rows."""
    sums, n_sums, eps = _norm_args(norm, x)
    width = qkv_shapes("gemm_stream_qkv", x, w, n_q_heads, n_kv_heads, head_dim, rotary_dim, cos_sin, k_pages, v_pages, slot_mapping, page_size)
    m, k = x.shape
    out = torch.empty((m, width), dtype=torch.bfloat16, device=x.device)
    check(
        core().tl_gemm_stream_qkv(
            x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0), m, k,
            n_q_heads, n_kv_heads, head_dim, rotary_dim, _ptr(cos_sin), _ptr(k_pages), _ptr(v_pages),
            _ptr(slot_mapping), page_size, waves, sums, n_sums, eps, _stream(),
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
#: Shapes never measured follow the size rule of ``linear_choice``.
LINEAR_CHOICE: dict = {}
ROW_BUCKETS = (1, 2, 4, 8, 16, 32, 64, 128)
STREAM_WAVE_CHOICES = (0, 4)
#: (strips per wave, splits of K, buffers) that ``tune_linear`` tries from 17 rows on: whole-K
#: launches for matrices with many rows, splits of K for those with few
WIDE_CHOICES = ((1, 1, 3), (2, 1, 3), (2, 1, 2), (1, 2, 3), (1, 4, 3), (2, 4, 3), (2, 4, 2), (1, 8, 3), (2, 8, 3), (2, 8, 2))


def wide_fits(rows: int, strips_per_wave: int, stages: int) -> bool:
    """Whether the buffers of such a launch fit the device's LDS (160 KB on gfx950): a buffer holds
    4 KB for every 16 rows of the row tile (32, 64 or 128) and 16 KB for every strip per wave."""
    tile = 32 if rows <= 32 else 64 if rows <= 64 else 128
    return stages * (tile // 16 * 4 + strips_per_wave * 16) * 1024 <= device_facts()[1]

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
TAIL_KERNEL_US = 2.8


def row_bucket(m: int) -> int:
    for b in ROW_BUCKETS:
        if m <= b:
            return b
    return ROW_BUCKETS[-1]


def fuses_tail(choice, use: str) -> bool:
    """Whether the kernel of ``choice`` does the second half of ``use`` itself.  For "sum" that half is the
    sum with the residual rows and the statistics of the norm behind it: the streaming kernel does both
    (``PendingProduct``), a split product leaves its slices to the norm kernel that runs anyway, the library
    needs that kernel where the streaming product would not."""
    if use == "plain":
        return True
    if choice is None:
        return False
    if choice[0] == "stream" or use == "sum":
        return True
    return choice[2] == 1 if use == "glu" else choice[2] > 1  # the gate ends a whole product, the rotation a split one


def linear_choice(x: torch.Tensor, w: torch.Tensor, use: str = "plain"):
    """Which bfloat16 kernel runs ``x @ w.T``: a tuple as in the table above, or None for the library.
    What the table holds decides.  A shape it does not hold follows a fixed rule: up to 16 rows the
    weight-streaming kernel (its own choice of waves) for matrices of at most ``STREAM_MAX_ELEMENTS``
    elements, the library otherwise."""
    m = x.shape[0]
    if m <= STREAM_MAX_ROWS:
        if not stream_supported(x, w):
            return None
        key = (w.shape[0], w.shape[1], row_bucket(m), use)
        if key in LINEAR_CHOICE:
            return LINEAR_CHOICE[key]
        return ("stream", 0) if w.shape[0] * w.shape[1] <= STREAM_MAX_ELEMENTS else None
    if not wide_supported(x, w):
        return None
    return LINEAR_CHOICE.get((w.shape[0], w.shape[1], row_bucket(m), use))


# ----------------------------------------------------------------------------- the table, outside the process
def kernel_table(shapes=None) -> dict:
    """The table as a JSON-able dict: ``"n,k,rows,use" -> choice`` (a list, or None for the library).
    ``shapes``: only the entries of these ``((n, k), use)`` pairs."""
    wanted = None if shapes is None else {(tuple(shape), use) for shape, use in shapes}
    out = {}
    for (n, k, bucket, use), choice in sorted(LINEAR_CHOICE.items(), key=lambda kv: (kv[0][0], kv[0][1], kv[0][3], kv[0][2])):
        if wanted is None or ((n, k), use) in wanted:
            out[f"{n},{k},{bucket},{use}"] = None if choice is None else list(choice)
    return out


def load_kernel_table(table) -> None:
    """Put the entries of ``table`` (a dict as ``kernel_table`` returns, or the path of a JSON file
    holding one) into the table; they replace what was measured for the same keys, and
    ``tune_linear`` leaves them alone.  Every entry is checked: a table from somewhere else must not
    be able to ask a kernel for a launch it does not have."""
    import json
    import os

    if isinstance(table, (str, os.PathLike)):
        with open(table) as f:
            table = json.load(f)
    entries = {}
    for key, choice in table.items():
        try:
            n, k, bucket, use = key.split(",")
            n, k, bucket = int(n), int(k), int(bucket)
        except ValueError:
            raise ValueError(f'kernel table: key {key!r} is not "n,k,rows,use"') from None
        if bucket not in ROW_BUCKETS or use not in LINEAR_USES or n <= 0 or k <= 0:
            raise ValueError(f"kernel table: key {key!r} names no row bucket {ROW_BUCKETS} or use {LINEAR_USES}")
        if choice is not None:
            choice = tuple(choice)
            ok = False
            if choice and choice[0] == "stream" and bucket <= STREAM_MAX_ROWS:
                ok = len(choice) in (2, 3) and choice[1] in STREAM_WAVE_CHOICES and (len(choice) == 2 or (use == "glu" and choice[2] in (8, 16)))
            elif choice and choice[0] == "wide" and bucket > STREAM_MAX_ROWS:
                ok = len(choice) == 4 and choice[1:] in WIDE_CHOICES and k % 128 == 0 and choice[2] <= k // 128 and wide_fits(bucket, choice[1], choice[3])
            if not ok:
                raise ValueError(f"kernel table: entry {key!r} -> {list(choice)!r} names no launch of a kernel here")
        entries[(n, k, bucket, use)] = choice
    LINEAR_CHOICE.update(entries)


def save_kernel_table(path, shapes=None) -> None:
    import json

    with open(path, "w") as f:
        json.dump(kernel_table(shapes), f, indent=1)


def clear_kernel_table() -> None:
    """Forget every measurement (the next ``tune_linear`` measures again)."""
    LINEAR_CHOICE.clear()


TUNE_FLUSH_BYTES = 512 << 20  # twice the 256 MB of last-level cache


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
    cannot take rotation and cache write into itself is charged the kernel that has to follow it, as is
    the library for "sum" at up to 16 rows, where the streaming kernel saves the norm's kernel.

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
    if all((n, k, bucket, use) in LINEAR_CHOICE for bucket in ROW_BUCKETS):
        return
    device = weights[0].device
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    # read, not written, before every replay: written lines would still be on their way to HBM
    # while the products are timed
    flush = torch.zeros(TUNE_FLUSH_BYTES // 4, dtype=torch.float32, device=device)  # (summed without a conversion pass)

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
        # (for "sum" only where the streaming kernel is a candidate: beyond its rows the norm kernel runs whoever multiplies)
        charged = use == "qkv" or (use == "sum" and bucket <= STREAM_MAX_ROWS and n % 4 == 0)
        tail = TAIL_KERNEL_US * 1e-3 * iters if charged and not fuses_tail(choice, use) else 0.0
        t = clock(fn) + tail
        if report is not None:
            report(bucket, choice, t / iters * 1e3)
        return t

    for bucket in ROW_BUCKETS:
        if (n, k, bucket, use) in LINEAR_CHOICE:
            continue
        x = torch.randn((bucket, k), device=device, dtype=torch.float32).to(torch.bfloat16)

        def run(choice):
            if use == "glu":
                return lambda w: run_glu(choice, x, w)
            return lambda w: run_choice(choice, x, w, out_dtype, leave_split=use == "sum")

        timed = [(None, cost(bucket, None, run(None)))]
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
        timed += [(choice, cost(bucket, choice, run(choice))) for choice in candidates]
        LINEAR_CHOICE[(n, k, bucket, use)] = pick(timed, use)


#: two candidates whose times differ by less than this share are taken to be equal: which of them a stopwatch
#: puts first changes from run to run (the library's product with a rotary kernel behind it against the split
#: product that rotates in its second kernel, at 64 rows of the 8B shape, did), and with it the bfloat16 bits
TUNE_TIE = 0.04


def pick(timed, use: str):
    """The choice among ``[(choice, time)]``: the fastest, except that among those within ``TUNE_TIE`` of the
    fastest one that does the whole of ``use`` in its own kernels comes before one that does not, and a kernel
    of this package before the library; among equals the first in the list (the candidates' fixed order)."""
    least = min(t for _, t in timed)
    close = [c for c, t in timed if t <= least * (1.0 + TUNE_TIE)]
    close.sort(key=lambda c: (not fuses_tail(c, use), c is None))  # (a stable sort: the list's order breaks ties)
    return close[0]


def run_choice(choice, x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, leave_split: bool = False):
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
    return run_choice(linear_choice(x, w), x, w, out_dtype)


def linear_to_sum(x: torch.Tensor, w: torch.Tensor, may_wait: bool = False):
    """``x @ w.T`` for a result that is only ever added to the residual stream by a norm's
    ``forward_add`` (after its ``delta(...)``) or by ``rmsnorm(..., delta=...)``: a tensor, or
    ``SplitSums`` when the product was split along K, which that ``rmsnorm`` adds up while it reads
    them.  With ``may_wait`` the product of the weight-streaming kernel is not run at all but handed
    on as a ``PendingProduct``, so that the kernel can add it to the residual stream itself."""
    if x.dtype == torch.float32:
        return gemm_f32(x, w)
    _gpu(x, w)
    choice = linear_choice(x, w, "sum")
    if may_wait and choice is not None and choice[0] == "stream" and w.dtype == torch.bfloat16 and w.shape[0] % 4 == 0:
        return PendingProduct(x, w, choice[1])
    return run_choice(choice, x, w, x.dtype, leave_split=True)


def linear_glu(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``silu(x @ gate.T) * (x @ up.T)`` for ``w`` [2F, K] = gate rows | up rows: one fused kernel
    where one of the decode kernels serves the shape, else the product followed by the gate.  ``x``
    may be ``NormedRows``: the weight-streaming kernel applies them, for any other they are normed first."""
    if isinstance(x, NormedRows):
        choice = linear_choice(x.gained, w, "glu")
        if choice is not None and choice[0] == "stream":
            return gemm_stream_glu(x.gained, w, choice[1], choice[2] if len(choice) > 2 else 16, norm=x)
        x = x.resolve()
    if x.dtype != torch.bfloat16:
        return silu_mul(linear(x, w))
    _gpu(x, w)
    return run_glu(linear_choice(x, w, "glu"), x, w)


def run_glu(choice, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    if choice is not None and choice[0] == "stream":
        return gemm_stream_glu(x, w, choice[1], choice[2] if len(choice) > 2 else 16)
    if choice is not None and choice[0] == "wide" and choice[2] == 1:
        return gemm_wide_glu(x, w, choice[1], choice[3])
    return silu_mul(run_choice(choice, x, w, x.dtype))


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
    multiple of 4), else product, bias and rotary kernels in turn.  ``x`` may be ``NormedRows``: the
    weight-streaming kernel applies them, for any other they are normed first."""
    norm = None
    if isinstance(x, NormedRows):
        norm, x = x, x.gained
        choice = linear_choice(x, w, "qkv")
        fusable = bias is None and head_dim % 4 == 0 and (rotary_dim == 0 or (pairing == 0 and cos_sin is not None))
        if not (fusable and choice is not None and choice[0] == "stream"):
            norm, x = None, norm.resolve()
    if x.dtype == torch.bfloat16:
        _gpu(x, w)
        choice = linear_choice(x, w, "qkv")
        fusable = bias is None and head_dim % 4 == 0 and (rotary_dim == 0 or (pairing == 0 and cos_sin is not None))
        if fusable and choice is not None and choice[0] == "stream":
            return gemm_stream_qkv(
                x, w, n_q_heads, n_kv_heads, head_dim, rotary_dim, cos_sin, k_pages, v_pages, slot_mapping, page_size, choice[1],
                norm=norm,
            )
        # (a product that is not split ends without a second kernel, so the rotary kernel follows it)
        if fusable and choice is not None and choice[0] == "wide" and choice[2] > 1:
            return gemm_wide_qkv(
                x, w, n_q_heads, n_kv_heads, head_dim, rotary_dim, cos_sin, k_pages, v_pages, slot_mapping, page_size,
                choice[1], choice[2], choice[3],
            )
        qkv = run_choice(choice, x, w, x.dtype)
    else:
        qkv = linear(x, w)
    if bias is not None:
        add_bias_(qkv, bias)
    rope_kv_write(
        qkv, n_q_heads, n_kv_heads, head_dim, positions, inv_freq, rotary_dim, pairing, k_pages, v_pages,
        slot_mapping, page_size, cos_sin=cos_sin,
    )
    return qkv
