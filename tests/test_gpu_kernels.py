"""Each kernel alone against its plain reference, at other sizes than the engine tests use."""

import math

import pytest
import torch
import torch.nn.functional as F

from .plain import llama as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def _ops():
    from torchllms_amd.kernels import ops

    return ops


class _Products:
    """The matrix products' own module (its table of measured choices), imported on first use."""

    def __getattr__(self, name):
        from torchllms_amd.kernels import products as module

        return getattr(module, name)


products = _Products()


def _i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


def _close_bf16(got, want, frac=0.002):
    """bfloat16 results may differ from the plain ones by one rounding in a few places."""
    got, want = got.float(), want.float()
    bad = (got - want).abs() > (want.abs() * 2 ** -7 + 1e-6)
    assert bad.float().mean().item() <= frac, f"{int(bad.sum())} of {bad.numel()} entries are off by more than one rounding"
    assert torch.allclose(got, want, rtol=2 ** -6, atol=1e-5)


# ----------------------------------------------------------------------------- embedding
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [72, 128, 1001])
def test_embed(dtype, hidden):
    torch.manual_seed(0)
    table = torch.randn(1000, hidden).to(dtype).to(DEV)
    toks = torch.randint(0, 1000, (37,), dtype=torch.int32, device=DEV)
    assert torch.equal(_ops().embed(toks, table), table[toks.long()])


# ----------------------------------------------------------------------------- RMS norm
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden, eps", [(100, 1e-5), (4096, 1e-6), (5000, 3e-4)])
def test_rmsnorm(dtype, hidden, eps):
    torch.manual_seed(0)
    x = (torch.randn(9, hidden) * 3).to(dtype)
    w = (1 + 0.2 * torch.randn(hidden)).to(dtype)
    got = _ops().rmsnorm(x.to(DEV), w.to(DEV), eps).cpu()
    want = plain.rms_norm(x, w, eps)
    if dtype == torch.float32:
        assert torch.allclose(got, want, rtol=2e-6, atol=1e-6)
    else:
        _close_bf16(got, want)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_with_residual_sum_rows_and_eps(dtype):
    torch.manual_seed(1)
    h = torch.randn(12, 320).to(dtype)
    d = torch.randn(12, 320).to(dtype)
    w = (1 + 0.2 * torch.randn(320)).to(dtype)
    s, y = _ops().rmsnorm(h.to(DEV), w.to(DEV), 1e-5, delta=d.to(DEV), return_sum=True)
    assert torch.equal(s.cpu(), h + d)  # the sum is rounded once, as an addition in the model's dtype
    want = plain.rms_norm(h + d, w, 1e-5)
    _close_bf16(y.cpu(), want) if dtype == torch.bfloat16 else torch.testing.assert_close(y.cpu(), want, rtol=2e-6, atol=1e-6)
    rows = _i32([7, 0, 7, 11])
    y2 = _ops().rmsnorm(h.to(DEV), w.to(DEV), 1e-5, delta=d.to(DEV), rows=rows).cpu()
    assert torch.equal(y2, y.cpu()[[7, 0, 7, 11]])
    # eps sits inside the root: a tiny row tells 1e-5 from 1e-6
    tiny = torch.full((1, 64), 1e-3).to(dtype).to(DEV)
    one = torch.ones(64, dtype=dtype, device=DEV)
    a = _ops().rmsnorm(tiny, one, 1e-5)[0, 0].item()
    b = _ops().rmsnorm(tiny, one, 1e-6)[0, 0].item()
    c = float(tiny[0, 0])
    assert a == pytest.approx(c / math.sqrt(c * c + 1e-5), rel=1e-2) and b == pytest.approx(c / math.sqrt(c * c + 1e-6), rel=1e-2)
    assert abs(a - b) > 0.1


def test_rmsnorm_weight_kept_in_32_bit():
    torch.manual_seed(2)
    x = torch.randn(4, 96).bfloat16()
    w = 1 + 0.2 * torch.randn(96)
    got = _ops().rmsnorm(x.to(DEV), w.to(DEV), 1e-5).cpu()
    xf = x.float()
    n = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)).bfloat16()
    _close_bf16(got, (n.float() * w).bfloat16())


# ----------------------------------------------------------------------------- rotary + cache write
def _pages(n_pages, hkv, page, dh, dtype):
    return (torch.zeros(n_pages, hkv, page, dh, dtype=dtype, device=DEV), torch.zeros(n_pages, hkv, page, dh, dtype=dtype, device=DEV))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq, hkv, dh, page", [(6, 3, 48, 4), (5, 5, 16, 16), (8, 1, 128, 32)])
def test_rope_and_cache_write(dtype, hq, hkv, dh, page):
    torch.manual_seed(0)
    n = 23
    qkv = torch.randn(n, (hq + 2 * hkv) * dh).to(dtype)
    pos = torch.randint(0, 500, (n,))
    inv_freq = plain.rope_inverse_frequencies(dh, 10000.0, None)
    n_pages = 12
    perm = torch.randperm(n_pages * page)[:n]  # every token a slot of its own, scattered over the pages
    k_pages, v_pages = _pages(n_pages, hkv, page, dh, dtype)
    dev = qkv.to(DEV)
    _ops().rope_kv_write(dev, hq, hkv, dh, _i32(pos.tolist()), inv_freq.to(DEV), dh, 0, k_pages, v_pages, _i32(perm.tolist()), page)
    q = qkv[:, : hq * dh].view(n, hq, dh)
    k = qkv[:, hq * dh : (hq + hkv) * dh].view(n, hkv, dh)
    v = qkv[:, (hq + hkv) * dh :].view(n, hkv, dh)
    want_q = plain.rope_rotate_interleaved(q, pos, inv_freq)
    want_k = plain.rope_rotate_interleaved(k, pos, inv_freq)
    tol = dict(rtol=1e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2 ** -7, atol=1e-3)
    torch.testing.assert_close(dev[:, : hq * dh].cpu().view(n, hq, dh), want_q, **tol)
    got_k = torch.stack([k_pages[s // page, :, s % page].cpu() for s in perm.tolist()])
    got_v = torch.stack([v_pages[s // page, :, s % page].cpu() for s in perm.tolist()])
    torch.testing.assert_close(got_k, want_k, **tol)
    assert torch.equal(got_v, v)  # values are stored as they are
    # nothing else was touched
    mask = torch.ones(n_pages * page, dtype=torch.bool)
    mask[perm] = False
    flat_k = k_pages.permute(0, 2, 1, 3).reshape(n_pages * page, hkv, dh).cpu()
    assert flat_k[mask].abs().sum() == 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_rope_half_pairing_partial_rotary_and_no_pages(dtype):
    torch.manual_seed(0)
    n, hq, hkv, dh, rot = 7, 3, 1, 32, 16
    qkv = torch.randn(n, (hq + 2 * hkv) * dh).to(dtype)
    pos = torch.arange(3, 3 + n)
    inv_freq = plain.rope_inverse_frequencies(rot, 100.0, None)
    dev = qkv.to(DEV)
    _ops().rope_kv_write(dev, hq, hkv, dh, _i32(pos.tolist()), inv_freq.to(DEV), rot, 1)
    heads = qkv.view(n, hq + 2 * hkv, dh)
    want = heads.clone()
    want[:, : hq + hkv, :rot] = plain.rope_rotate_half_split(heads[:, : hq + hkv, :rot], pos, inv_freq)
    tol = dict(rtol=1e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2 ** -7, atol=1e-3)
    torch.testing.assert_close(dev.cpu().view(n, hq + 2 * hkv, dh), want, **tol)  # k rotated in place, v and the tail untouched
    # rotary_dim 0: nothing moves
    dev = qkv.to(DEV)
    _ops().rope_kv_write(dev, hq, hkv, dh, _i32(pos.tolist()), None, 0, 0)
    assert torch.equal(dev.cpu(), qkv)


def test_rope_table_and_its_use_give_what_the_kernel_computes_itself():
    torch.manual_seed(0)
    n, hq, hkv, dh, rot = 9, 4, 2, 32, 24
    pos = torch.tensor([0, 1, 7, 500, 8191, 131071, 3, 3, 12])
    inv_freq = plain.rope_inverse_frequencies(rot, 500000.0, None)
    table = _ops().rope_table(_i32(pos.tolist()), inv_freq.to(DEV))
    ang = pos.float()[:, None] * inv_freq[None, :]  # 32-bit product, as the reference's table
    torch.testing.assert_close(table[..., 0].cpu(), torch.cos(ang), rtol=0, atol=2e-7)
    torch.testing.assert_close(table[..., 1].cpu(), torch.sin(ang), rtol=0, atol=2e-7)
    for dtype in DTYPES:
        qkv = torch.randn(n, (hq + 2 * hkv) * dh).to(dtype)
        a, b = qkv.to(DEV), qkv.to(DEV)
        _ops().rope_kv_write(a, hq, hkv, dh, _i32(pos.tolist()), inv_freq.to(DEV), rot, 0)
        _ops().rope_kv_write(b, hq, hkv, dh, _i32(pos.tolist()), None, rot, 0, cos_sin=table)
        # the table takes the wide-access kernel: the same cosines and sines, products possibly
        # fused differently, so equal but for the last bit
        tol = dict(rtol=2e-7, atol=1e-6) if dtype == torch.float32 else dict(rtol=2 ** -8, atol=1e-6)
        torch.testing.assert_close(a.float(), b.float(), **tol)
        assert (a != b).float().mean().item() < 0.02
        # half-split pairing keeps the narrow kernel, table or not: bit-equal
        a, b = qkv.to(DEV), qkv.to(DEV)
        _ops().rope_kv_write(a, hq, hkv, dh, _i32(pos.tolist()), inv_freq.to(DEV), rot, 1)
        _ops().rope_kv_write(b, hq, hkv, dh, _i32(pos.tolist()), None, rot, 1, cos_sin=table)
        assert torch.equal(a, b)


@pytest.mark.parametrize("m, hq, hkv, dh, rot, page, k", [(8, 32, 8, 128, 128, 16, 4096), (1, 4, 4, 64, 64, 16, 256),
                                                           (13, 6, 3, 48, 24, 4, 136), (16, 5, 1, 20, 0, 8, 64), (3, 2, 2, 16, 16, 2, 8)])
@pytest.mark.parametrize("with_pages", [True, False])
def test_gemm_stream_qkv_equals_product_then_rotary_kernel(m, hq, hkv, dh, rot, page, k, with_pages):
    """The fused projection against the two kernels it replaces, on every output: rotated queries
    in the buffer, rotated keys and raw values in their pages (or in the buffer without pages);
    a row whose slot is negative stores nothing."""
    torch.manual_seed(2)
    width = (hq + 2 * hkv) * dh
    x = torch.randn(m, k).bfloat16().to(DEV)
    w = (torch.randn(width, k) * k ** -0.5).bfloat16().to(DEV)
    pos = torch.randint(0, 9000, (m,))
    inv_freq = plain.rope_inverse_frequencies(rot, 500000.0, None).to(DEV) if rot else None
    table = _ops().rope_table(_i32(pos.tolist()), inv_freq) if rot else None
    n_pages = 40
    slots = torch.randperm(n_pages * page)[:m].tolist()
    if m > 2:
        slots[1] = -1
    outs = []
    for fused in (False, True):
        kp, vp = _pages(n_pages, hkv, page, dh, torch.bfloat16) if with_pages else (None, None)
        sm = _i32(slots) if with_pages else None
        if fused:
            qkv = _ops().gemm_stream_qkv(x, w, hq, hkv, dh, rot, table, kp, vp, sm, page if with_pages else 0)
        else:
            qkv = _ops().gemm_stream(x, w)
            _ops().rope_kv_write(qkv, hq, hkv, dh, _i32(pos.tolist()), inv_freq, rot, 0, kp, vp, sm, page if with_pages else 0, cos_sin=table)
        outs.append((qkv, kp, vp))
    (qa, ka, va), (qb, kb, vb) = outs
    cols = hq * dh if with_pages else width  # with pages only the queries of the buffer are defined
    tol = dict(rtol=2 ** -7, atol=2 ** -8 * qa.float().abs().max().item())
    torch.testing.assert_close(qb[:, :cols].float(), qa[:, :cols].float(), **tol)
    assert (qb[:, :cols] != qa[:, :cols]).float().mean().item() < 0.05  # only last-bit differences of the sums
    if with_pages:
        torch.testing.assert_close(kb.float(), ka.float(), **tol)
        torch.testing.assert_close(vb.float(), va.float(), **tol)
        assert (kb.float().abs().sum(dim=(1, 3)) > 0).sum().item() == m - (1 if m > 2 else 0)  # one slot per stored row


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq, hkv, dh, rot, page", [(32, 8, 128, 128, 16), (6, 3, 48, 20, 4), (5, 5, 16, 16, 16), (3, 1, 24, 0, 8)])
def test_rope_wide_kernel_with_table_and_pages(dtype, hq, hkv, dh, rot, page):
    """The kernel the engine's prefill takes (table of cosines, 16-byte accesses): queries in place,
    rotated keys and raw values in their pages, partial rotary cut inside a 16-byte piece, a
    token without a slot stores nothing."""
    torch.manual_seed(0)
    n = 37
    qkv = torch.randn(n, (hq + 2 * hkv) * dh).to(dtype)
    pos = torch.randint(0, 9000, (n,))
    inv_freq = plain.rope_inverse_frequencies(rot, 500000.0, None) if rot else None
    table = _ops().rope_table(_i32(pos.tolist()), inv_freq.to(DEV)) if rot else None
    n_pages = 12
    slots = torch.randperm(n_pages * page)[:n].tolist()
    slots[5] = -1
    k_pages, v_pages = _pages(n_pages, hkv, page, dh, dtype)
    dev = qkv.to(DEV)
    _ops().rope_kv_write(dev, hq, hkv, dh, _i32(pos.tolist()), None, rot, 0, k_pages, v_pages, _i32(slots), page, cos_sin=table)
    heads = qkv.view(n, hq + 2 * hkv, dh)
    want = heads.clone().float()
    if rot:
        want[:, : hq + hkv, :rot] = plain.rope_rotate_interleaved(heads[:, : hq + hkv, :rot], pos, inv_freq)
    tol = dict(rtol=1e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2 ** -7, atol=1e-3)
    torch.testing.assert_close(dev.cpu().view(n, hq + 2 * hkv, dh)[:, :hq].float(), want[:, :hq], **tol)
    for i, s in enumerate(slots):
        if s < 0:
            continue
        torch.testing.assert_close(k_pages[s // page, :, s % page].cpu().float(), want[i, hq : hq + hkv], **tol)
        assert torch.equal(v_pages[s // page, :, s % page].cpu(), heads[i, hq + hkv :])
    stored = (k_pages.float().abs().sum(dim=(1, 3)) > 0).sum().item()
    assert stored == n - 1


def test_cache_write_round_trip_with_distinct_values():
    # reference: torchllms/models/test_paged_kv.py:440-484 (append then extract, value = position)
    hq, hkv, dh, page = 2, 2, 8, 4
    n = 11
    qkv = torch.zeros(n, (hq + 2 * hkv) * dh, dtype=torch.bfloat16)
    for p in range(n):
        qkv[p, hq * dh : (hq + hkv) * dh] = p + 1
        qkv[p, (hq + hkv) * dh :] = -(p + 1)
    k_pages, v_pages = _pages(5, hkv, page, dh, torch.bfloat16)
    table = [3, 0, 4]
    slots = [table[p // page] * page + p % page for p in range(n)]
    _ops().rope_kv_write(qkv.to(DEV), hq, hkv, dh, _i32(list(range(n))), None, 0, 0, k_pages, v_pages, _i32(slots), page)
    for p in range(n):
        assert (k_pages[table[p // page], :, p % page] == p + 1).all()
        assert (v_pages[table[p // page], :, p % page] == -(p + 1)).all()


# ----------------------------------------------------------------------------- SwiGLU gate, bias
@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(dtype):
    torch.manual_seed(0)
    gu = (torch.randn(5, 2 * 203) * 3).to(dtype)
    got = _ops().silu_mul(gu.to(DEV)).cpu()
    want = F.silu(gu[:, :203]) * gu[:, 203:]
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, rtol=2e-6, atol=1e-6)
    else:
        _close_bf16(got, want)


@pytest.mark.parametrize("dtype", DTYPES)
def test_add_bias(dtype):
    torch.manual_seed(0)
    x = torch.randn(6, 50).to(dtype)
    b = torch.randn(30).to(dtype)
    got = _ops().add_bias_(x.to(DEV), b.to(DEV)).cpu()
    want = x.clone()
    want[:, :30] = x[:, :30] + b
    assert torch.equal(got, want)


# ----------------------------------------------------------------------------- 32-bit matrix product
@pytest.mark.parametrize("m, n, k", [(1, 100, 50), (7, 257, 1000), (130, 64, 64), (65, 129, 17), (300, 391, 70), (97, 130, 1029)])
def test_gemm_f32_is_true_32_bit(m, n, k):
    torch.manual_seed(0)
    x, w = torch.randn(m, k), torch.randn(n, k)
    got = _ops().gemm_f32(x.to(DEV), w.to(DEV)).cpu()
    want = (x.double() @ w.double().T)
    assert (got.double() - want).abs().max().item() < 2e-6 * math.sqrt(k) * 4
    # a row's result does not depend on the rows beside it
    alone = _ops().gemm_f32(x[:1].to(DEV), w.to(DEV)).cpu()
    assert torch.equal(alone[0], got[0])


@pytest.mark.parametrize("n, k", [(64, 4096), (50, 1030), (4099, 100), (16, 14336), (33, 16), (7, 5)])
def test_gemm_f32_with_few_rows_gives_the_bits_of_the_kernel_for_many(n, k):
    """Up to 16 rows (decode steps) take a kernel that spreads an element's groups of 16 products over
    the lanes of a wave and adds their sums in the groups' order: the same arithmetic per element as the
    tiled kernel for more rows, so the same bits, whatever the number of rows, also where K is no
    multiple of 16 or of a round of 1,024, N no multiple of 16, and rows are strided."""
    torch.manual_seed(n + k)
    x = torch.randn(40, k + 3)[:, :k].to(DEV)  # rows with a stride that is no multiple of 4
    w = torch.randn(n, k).to(DEV)
    many = _ops().gemm_f32(x, w)  # 40 rows: the tiled kernel
    want = x.double() @ w.double().T
    assert (many.double() - want).abs().max().item() < 2e-6 * math.sqrt(k) * 4
    for rows in (1, 2, 3, 4, 7, 8, 13, 16):
        few = _ops().gemm_f32(x[:rows], w)
        assert torch.equal(few, many[:rows]), f"{rows} rows differ from the tiled kernel"
    shifted = _ops().gemm_f32(x[5:8], w)
    assert torch.equal(shifted, many[5:8])
    # prompts take a larger tile with more of the result per thread: the same sums again
    torch.manual_seed(n + k + 1)
    tall = torch.cat([x, torch.randn(131, k + 3, device=DEV)[:, :k]])
    assert torch.equal(_ops().gemm_f32(tall, w)[:40], many)
    assert torch.equal(_ops().gemm_f32(tall[37:], w)[:3], many[37:])
    if k % 4 == 0:
        aligned = _ops().gemm_f32(x[:2].contiguous(), w)
        assert torch.equal(aligned, many[:2])


# ----------------------------------------------------------------------------- attention
def _paged(k, v, page, n_pages, seed=0, dtype=torch.float32):
    """Scatter dense per-request keys/values [S, Hkv, dh] into shuffled pages; returns pages and
    the block table."""
    S, hkv, dh = k.shape
    g = torch.Generator().manual_seed(seed)
    n_blocks = -(-S // page)
    table = torch.randperm(n_pages, generator=g)[:n_blocks].tolist()
    # unused pages hold large values: reading one shows
    k_pages = torch.full((n_pages, hkv, page, dh), 50.0, dtype=dtype)
    v_pages = torch.full((n_pages, hkv, page, dh), -50.0, dtype=dtype)
    for p in range(S):
        k_pages[table[p // page], :, p % page] = k[p]
        v_pages[table[p // page], :, p % page] = v[p]
    return k_pages.to(DEV), v_pages.to(DEV), table


def _attend(fn, q, k, v, page, window=0, q_start=None, scale=None, dtype=torch.float32, n_pages=None):
    """Run ``fn`` (a kernel wrapper) for the queries ``q`` [Sq, Hq, dh], which are the last Sq
    positions of a request whose keys/values are ``k``, ``v`` [S, Hkv, dh]."""
    sq, hq, dh = q.shape
    S, hkv, _ = k.shape
    n_pages = n_pages or (-(-S // page) + 3)
    k_pages, v_pages, table = _paged(k.to(dtype), v.to(dtype), page, n_pages, dtype=dtype)
    q_start = S - sq if q_start is None else q_start
    qkv = q.reshape(sq, hq * dh).to(dtype).to(DEV).contiguous()
    out = fn(
        qkv, hq, hkv, dh, k_pages, v_pages, _i32([0] * sq), _i32(list(range(q_start, q_start + sq))), _i32([table]),
        window, scale if scale is not None else dh ** -0.5,
    )
    return out.float().cpu()


def _windowed_plain(q, k, v, window):
    """The plain attention, one query at a time over the keys its window leaves."""
    sq = q.shape[0]
    S = k.shape[0]
    rows = []
    for i in range(sq):
        p = S - sq + i
        lo = max(p - window + 1, 0) if window > 0 else 0
        rows.append(plain.attention(q[i : i + 1], k[lo : p + 1], v[lo : p + 1]))
    return torch.cat(rows)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize(
    "hq, hkv, dh, page, S, sq",
    [(4, 2, 16, 8, 37, 37), (6, 3, 48, 4, 150, 9), (8, 1, 128, 16, 300, 1), (3, 3, 80, 32, 70, 70), (2, 1, 256, 16, 65, 2), (4, 4, 64, 1, 20, 20)],
)
def test_attention_generic(dtype, hq, hkv, dh, page, S, sq):
    torch.manual_seed(0)
    q = torch.randn(sq, hq, dh) * 2
    k = torch.randn(S, hkv, dh)
    v = torch.randn(S, hkv, dh)
    if dtype == torch.bfloat16:
        q, k, v = q.bfloat16().float(), k.bfloat16().float(), v.bfloat16().float()
    got = _attend(_ops().attention_generic, q, k, v, page, dtype=dtype)
    want = plain.attention(q, k, v)
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)
    else:
        torch.testing.assert_close(got, want, rtol=2 ** -7, atol=2 ** -7)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize(
    "hq, hkv, dh, page, sizes, window",
    [(8, 2, 128, 16, [(300, 200), (70, 70), (40, 3)], 0), (6, 3, 48, 4, [(150, 90), (33, 33)], 0), (4, 4, 64, 8, [(260, 100), (90, 40)], 37),
     (3, 1, 20, 5, [(100, 64), (50, 50)], 0), (16, 2, 256, 16, [(130, 50)], 100), (5, 5, 18, 3, [(80, 41)], 0)],
)
def test_attention_generic_for_prompt_portions_gives_the_bits_of_one_token_at_a_time(dtype, hq, hkv, dh, page, sizes, window):
    """Steps with many tokens bring each block of 64 keys into LDS once for sixteen (token, head) pairs that
    read it; the arithmetic per pair is the walk of a single wave, so the results are the same bits as when every
    token is a step of its own (which takes the kernel that shares nothing).  Requests of different lengths in
    one launch (blocks that straddle two requests walk alone), groups of 1, 2, 4 and 8 query heads per kv head,
    head sizes that are no multiple of 4, a window, right against the plain attention."""
    torch.manual_seed(dh + page)
    k_all, v_all, q_all, seqs, poss, tables = [], [], [], [], [], []
    n_pages = sum(-(-S // page) for S, _ in sizes) + 2
    perm = torch.randperm(n_pages).tolist()
    k_pages = torch.zeros(n_pages, hkv, page, dh, dtype=dtype)
    v_pages = torch.zeros_like(k_pages)
    width = max(-(-S // page) for S, _ in sizes)
    want = []
    for r, (S, sq) in enumerate(sizes):
        q = torch.randn(sq, hq, dh) * 2
        k, v = torch.randn(S, hkv, dh), torch.randn(S, hkv, dh)
        if dtype == torch.bfloat16:
            q, k, v = q.bfloat16().float(), k.bfloat16().float(), v.bfloat16().float()
        table = [perm.pop() for _ in range(-(-S // page))]
        for p_ in range(S):
            k_pages[table[p_ // page], :, p_ % page] = k[p_].to(dtype)
            v_pages[table[p_ // page], :, p_ % page] = v[p_].to(dtype)
        tables.append(table + [-1] * (width - len(table)))
        q_all.append(q.reshape(sq, hq * dh))
        seqs += [r] * sq
        poss += list(range(S - sq, S))
        want.append(_windowed_plain(q, k, v, window))
    qkv = torch.cat(q_all).to(dtype).to(DEV).contiguous()
    k_pages, v_pages = k_pages.to(DEV), v_pages.to(DEV)
    bt = _i32(tables)
    fn = _ops().attention_generic
    together = fn(qkv, hq, hkv, dh, k_pages, v_pages, _i32(seqs), _i32(poss), bt, window, dh ** -0.5)
    assert len(seqs) >= 32
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2 ** -7, atol=2 ** -7)
    torch.testing.assert_close(together.float().cpu(), torch.cat(want).reshape(len(seqs), hq * dh), **tol)
    for i in list(range(0, len(seqs), 7)) + [len(seqs) - 1]:
        alone = fn(qkv[i : i + 1], hq, hkv, dh, k_pages, v_pages, _i32(seqs[i : i + 1]), _i32(poss[i : i + 1]), bt, window, dh ** -0.5)
        assert torch.equal(alone[0], together[i]), f"token {i} differs from the same token alone"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize(
    "hq, hkv, dh, page, S, sq, window",
    [(4, 2, 16, 8, 37, 3, 0), (6, 3, 48, 4, 150, 9, 0), (8, 1, 128, 16, 700, 2, 0), (3, 3, 6, 32, 270, 5, 0), (2, 1, 256, 16, 65, 2, 0),
     (4, 4, 64, 1, 200, 4, 70), (5, 5, 32, 16, 1000, 3, 64), (2, 2, 80, 8, 129, 1, 0)],
)
def test_attention_generic_in_blocks_of_their_own_gives_the_same_bits(dtype, hq, hkv, dh, page, S, sq, window):
    """The plain kernel computes every block of 64 keys by itself and lets the blocks join in ascending
    order; for decode steps the blocks are computed by waves of their own and joined by a second
    kernel.  Same blocks, same operations, same order: the same bits, with a window and without, with
    head sizes that are no multiple of 4, and whatever the bound on the context says."""
    torch.manual_seed(5)
    q = torch.randn(sq, hq, dh) * 2
    k = torch.randn(S, hkv, dh)
    v = torch.randn(S, hkv, dh)
    one_wave = _attend(_ops().attention_generic, q, k, v, page, window=window, dtype=dtype)
    want = _windowed_plain(q, k, v, window)
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2 ** -6, atol=2 ** -6)
    if dtype == torch.bfloat16:
        want = _windowed_plain(q.bfloat16().float(), k.bfloat16().float(), v.bfloat16().float(), window)
    torch.testing.assert_close(one_wave, want, **tol)
    for longest in (S, S + 200, min(window, S) if window else S):
        def split(*a):
            return _ops().attention_generic_split(*a, longest=longest)

        many = _attend(split, q, k, v, page, window=window, dtype=dtype)
        assert torch.equal(many, one_wave), f"bound {longest}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_finds_a_far_key_among_hundreds(dtype):
    """One key far back matches the query; its value must come out.  A kernel that drops or
    misplaces a block of keys, or reads the wrong page, returns something else."""
    torch.manual_seed(0)
    hq, hkv, dh, page, S = 4, 2, 32, 16, 700
    k = torch.randn(S, hkv, dh) * 0.1
    v = torch.randn(S, hkv, dh)
    q = torch.randn(1, hq, dh) * 0.1
    for far in (0, 1, 15, 16, 63, 64, 65, 333, 639, 640, 698, 699):
        kk, qq = k.clone(), q.clone()
        direction = torch.randn(dh)
        direction /= direction.norm()
        kk[far, :, :] = direction * 12
        qq[0, :, :] = direction * 12 * math.sqrt(dh) / 4  # score 36 for that key, about 0 for all others
        got = _attend(_ops().attention_generic, qq, kk, v, page, dtype=dtype).view(hq, dh)
        want = v[far].repeat_interleave(hq // hkv, dim=0)
        tol = 1e-4 if dtype == torch.float32 else 2e-2
        assert (got - want).abs().max().item() < tol, f"key {far}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 5, 64, 100])
def test_attention_window_edge(dtype, window):
    """The key just outside the window is made to match the query: it must not be seen.  The one
    just inside is seen."""
    torch.manual_seed(0)
    hq, hkv, dh, page, S, sq = 2, 1, 16, 8, 230, 3
    k = torch.randn(S, hkv, dh) * 0.1
    v = torch.randn(S, hkv, dh)
    q = torch.randn(sq, hq, dh)
    want = _windowed_plain(q, k, v, window)
    got = _attend(_ops().attention_generic, q, k, v, page, window=window, dtype=dtype)
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2 ** -7, atol=2 ** -7)
    torch.testing.assert_close(got, want, **tol)
    p = S - 1
    direction = torch.ones(dh) / math.sqrt(dh)
    qq = q.clone()
    qq[-1] = direction * 40
    outside = p - window
    if outside >= 0:
        kk = k.clone()
        kk[outside, 0] = direction * 10
        got = _attend(_ops().attention_generic, qq, kk, v, page, window=window, dtype=dtype)
        torch.testing.assert_close(got[-1:], _windowed_plain(qq, kk, v, window)[-1:], **tol)
        assert (got[-1].view(hq, dh) - v[outside, 0]).abs().max() > 0.05
    inside = p - window + 1
    kk = k.clone()
    kk[inside, 0] = direction * 10
    got = _attend(_ops().attention_generic, qq, kk, v, page, window=window, dtype=dtype)
    assert (got[-1].view(hq, dh) - v[inside, 0]).abs().max() < (1e-3 if dtype == torch.float32 else 3e-2)


def test_attention_window_never_reads_released_pages():
    """Blocks wholly before the window are -1 in the block table; the kernel must not touch them."""
    torch.manual_seed(0)
    hq, hkv, dh, page, S, window = 2, 2, 16, 4, 60, 6
    q, k, v = torch.randn(1, hq, dh), torch.randn(S, hkv, dh), torch.randn(S, hkv, dh)
    k_pages, v_pages, table = _paged(k, v, page, 20)
    first_needed = (S - 1 - window + 1) // page
    table = [-1 if b < first_needed else t for b, t in enumerate(table)]
    out = _ops().attention_generic(
        q.reshape(1, hq * dh).to(DEV), hq, hkv, dh, k_pages, v_pages, _i32([0]), _i32([S - 1]), _i32([table]), window, dh ** -0.5
    ).cpu()
    torch.testing.assert_close(out, _windowed_plain(q, k, v, window), rtol=1e-5, atol=1e-5)


def test_attention_batch_of_requests_and_strided_queries():
    """Three requests in one launch, queries read out of a wider row (the fused q|k|v buffer)."""
    torch.manual_seed(0)
    hq, hkv, dh, page = 4, 2, 32, 8
    lens = [(21, 21), (50, 1), (33, 5)]  # (tokens cached, new queries)
    n_pages = 20
    k_pages = torch.zeros(n_pages, hkv, page, dh)
    v_pages = torch.zeros(n_pages, hkv, page, dh)
    free = torch.randperm(n_pages).tolist()
    tables, wants, qs, seq, pos = [], [], [], [], []
    for b, (S, sq) in enumerate(lens):
        k, v, q = torch.randn(S, hkv, dh), torch.randn(S, hkv, dh), torch.randn(sq, hq, dh)
        table = [free.pop() for _ in range(-(-S // page))]
        for p in range(S):
            k_pages[table[p // page], :, p % page] = k[p]
            v_pages[table[p // page], :, p % page] = v[p]
        tables.append(table + [-1] * (7 - len(table)))
        wants.append(plain.attention(q, k, v))
        qs.append(q.reshape(sq, hq * dh))
        seq += [b] * sq
        pos += list(range(S - sq, S))
    wide = torch.cat([torch.cat(qs), torch.randn(len(seq), 2 * hkv * dh)], dim=1).to(DEV)
    out = _ops().attention_generic(wide, hq, hkv, dh, k_pages.to(DEV), v_pages.to(DEV), _i32(seq), _i32(pos), _i32(tables), 0, dh ** -0.5)
    torch.testing.assert_close(out.cpu(), torch.cat(wants), rtol=1e-5, atol=1e-5)


def test_attention_refuses_sizes_it_does_not_have():
    from torchllms_amd.kernels.lib import KernelError

    q = torch.zeros(1, 2 * 272, device=DEV)
    pages = torch.zeros(2, 2, 4, 272, device=DEV)
    with pytest.raises(KernelError, match="head_dim=272"):
        _ops().attention_generic(q, 2, 2, 272, pages, pages, _i32([0]), _i32([0]), _i32([[0]]), 0, 1.0)
    q = torch.zeros(1, 3 * 16, device=DEV)
    pages = torch.zeros(2, 2, 4, 16, device=DEV)
    with pytest.raises(KernelError, match="not a multiple"):
        _ops().attention_generic(q, 3, 2, 16, pages, pages, _i32([0]), _i32([0]), _i32([[0]]), 0, 1.0)
    with pytest.raises(KernelError, match="GPU"):
        _ops().silu_mul(torch.zeros(2, 4))


# ----------------------------------------------------------------------------- sampling
def _sample(logits, temps, seeds, steps, top_k=None):
    n = logits.shape[0]
    return _ops().sample(
        logits.to(DEV), torch.tensor(temps, dtype=torch.float32, device=DEV), torch.tensor(seeds, dtype=torch.int64, device=DEV),
        torch.tensor(steps, dtype=torch.int64, device=DEV), None if top_k is None else _i32(top_k),
    ).cpu()


def test_sample_greedy_and_ties():
    torch.manual_seed(0)
    logits = torch.randn(5, 1003)
    logits[2, 77] = logits[2, 900] = 9.0  # the lowest index among equal maxima
    got = _sample(logits, [0.0] * 5, [1] * 5, [0] * 5)
    assert got.tolist() == logits.argmax(-1).tolist() and got[2] == 77


@pytest.mark.parametrize("vocab", [128256, 40000, 16388, 4099])
def test_sample_greedy_over_a_large_vocabulary(vocab):
    """Wide loads, their unrolled part, their tail and the unaligned rows of an odd vocabulary; the
    maximum is planted at the far end, at the start and twice (the lower index wins)."""
    torch.manual_seed(1)
    logits = torch.randn(6, vocab)
    logits[0, vocab - 1] = 50.0
    logits[1, 0] = 50.0
    logits[2, vocab - 3] = logits[2, 5] = 50.0
    mid = min(4 * 1024 * 3 + 2, vocab - 7)
    logits[3, mid] = logits[3, vocab - 2] = 50.0
    logits[4, vocab // 2 + 1] = 50.0
    got = _sample(logits, [0.0] * 6, [1] * 6, [0] * 6)
    assert got.tolist() == [vocab - 1, 0, 5, mid, vocab // 2 + 1, int(logits[5].argmax())]


@pytest.mark.parametrize("vocab", [8, 301, 5000])
def test_sample_temperature_matches_the_plain_rule(vocab):
    torch.manual_seed(0)
    logits = torch.randn(6, vocab) * 2
    logits[5] = logits[0]
    seeds, steps = [3, 3, 4, 5, 2 ** 40 + 7, 3], [0, 1, 0, 9, 2 ** 33, 0]
    got = _sample(logits, [0.7] * 6, seeds, steps)
    for r in range(6):
        u = _ops().philox_uniform(seeds[r], steps[r], vocab, DEV).cpu()
        assert (u > 0).all() and (u < 1).all()
        want = plain.sample_with_exponentials(logits[r], 0.7, -torch.log(u))
        assert got[r] == want
    assert got[0] == got[5]  # same seed and step: same draw, whatever the row
    # top-k: the draw comes from the k largest
    got = _sample(logits, [1.5] * 6, seeds, steps, top_k=[3] * 6)
    for r in range(6):
        assert got[r] in logits[r].topk(3).indices.tolist()
        u = _ops().philox_uniform(seeds[r], steps[r], vocab, DEV).cpu()
        assert got[r] == plain.sample_with_exponentials(logits[r], 1.5, -torch.log(u), top_k=3)


@pytest.mark.parametrize("vocab, rows", [(128256, 8), (128256, 64), (40000, 3), (16388, 5)])
def test_sample_with_several_blocks_a_row_draws_what_one_block_draws(vocab, rows):
    """Few rows of a large vocabulary are cut into pieces for blocks of their own (a vector of
    zeros as top-k keeps the one-block kernel): the same tokens, greedy rows and ties included,
    and the plain rule's token."""
    ops = _ops()
    assert ops.sample_chunks(rows, vocab) > 1 and ops.sample_chunks(512, vocab) == 1 and ops.sample_chunks(4, 5000) == 1
    torch.manual_seed(3)
    logits = torch.randn(rows, vocab) * 3
    logits[1, vocab - 1] = logits[1, 9000] = 40.0  # a tie across pieces in a greedy row
    temps = [0.7, 0.0, 1.3] + [0.9] * (rows - 3)
    seeds, steps = list(range(11, 11 + rows)), list(range(rows))
    many = _sample(logits, temps, seeds, steps)
    one = _sample(logits, temps, seeds, steps, top_k=[0] * rows)
    assert many.tolist() == one.tolist() and many[1] == 9000
    u = ops.philox_uniform(seeds[2], steps[2], vocab, DEV).cpu()
    assert many[2] == plain.sample_with_exponentials(logits[2], 1.3, -torch.log(u))


def test_sample_mixed_rows_and_tiny_temperature():
    torch.manual_seed(0)
    logits = torch.randn(4, 200)
    got = _sample(logits, [0.0, 1e-7, 0.9, 0.0], [5, 6, 7, 8], [0, 0, 0, 0])
    assert got[0] == logits[0].argmax() and got[1] == logits[1].argmax() and got[3] == logits[3].argmax()


def test_sample_frequencies_follow_softmax():
    logits = torch.tensor([1.0, 0.0, -1.0, 2.0, 0.5, -3.0])
    n = 20000
    got = _sample(logits.expand(n, 6).contiguous(), [0.7] * n, [123] * n, list(range(n)))
    freq = torch.bincount(got.long(), minlength=6).float()
    expect = torch.softmax(logits / 0.7, -1) * n
    chi2 = ((freq - expect) ** 2 / expect).sum().item()
    assert chi2 < 20.5  # 5 degrees of freedom, p = 0.001
    u = _ops().philox_uniform(9, 0, 100000, DEV).cpu()
    assert abs(u.mean().item() - 0.5) < 0.005 and abs(u.var().item() - 1 / 12) < 0.002


# ----------------------------------------------------------------------------- decode attention (MFMA, split-KV)
def _decode(q, k, v, page, window=0, split_size=None, n_pages=None):
    """The decode kernel for one token (the last position of the request) with bfloat16 inputs."""
    hq, dh = q.shape[1], q.shape[2]
    S, hkv, _ = k.shape
    n_pages = n_pages or (-(-S // page) + 3)
    k_pages, v_pages, table = _paged(k.bfloat16(), v.bfloat16(), page, n_pages, dtype=torch.bfloat16)
    qkv = q.reshape(1, hq * dh).bfloat16().to(DEV).contiguous()
    lo = max(S - window, 0) if window else 0
    longest = S - (lo // 16) * 16
    out = _ops().attention_decode(
        qkv, hq, hkv, dh, k_pages, v_pages, _i32([0]), _i32([S - 1]), _i32([table]), window, dh ** -0.5, longest, split_size=split_size
    )
    return out.float().cpu()


@pytest.mark.parametrize(
    "hq, hkv, dh, page, S, split",
    [
        (32, 8, 128, 16, 2000, None), (32, 8, 128, 16, 2000, 64), (32, 8, 128, 16, 2000, 4096), (8, 1, 32, 16, 300, 64),
        (4, 4, 64, 8, 100, None), (6, 2, 64, 4, 77, 64), (16, 1, 128, 32, 513, 128), (8, 1, 256, 16, 200, 64),
        (5, 5, 32, 12, 130, 64), (6, 3, 128, 1, 65, 64), (2, 2, 64, 16, 1, None), (4, 1, 128, 16, 16, None), (4, 1, 128, 16, 17, None),
        (4, 1, 128, 16, 5000, 64), (2, 1, 64, 16, 4500, 64),  # more than 64 splits: the merge reads statistics past its first wave of lanes
    ],
)
def test_attention_decode(hq, hkv, dh, page, S, split):
    torch.manual_seed(0)
    q = (torch.randn(1, hq, dh) * 2).bfloat16().float()
    k = torch.randn(S, hkv, dh).bfloat16().float()
    v = torch.randn(S, hkv, dh).bfloat16().float()
    got = _decode(q, k, v, page, split_size=split)
    want = plain.attention(q, k, v)
    torch.testing.assert_close(got, want, rtol=2 ** -7, atol=2 ** -7)


def test_attention_decode_finds_a_far_key_among_thousands():
    torch.manual_seed(0)
    hq, hkv, dh, page, S = 8, 2, 128, 16, 3000
    k = torch.randn(S, hkv, dh) * 0.1
    v = torch.randn(S, hkv, dh)
    for far in (0, 1, 15, 16, 17, 63, 64, 255, 256, 1000, 2047, 2048, 2998, 2999):
        kk = k.clone()
        direction = torch.randn(dh)
        direction /= direction.norm()
        kk[far] = direction * 12
        qq = (direction * 12 * math.sqrt(dh) / 4).expand(1, hq, dh).clone()
        got = _decode(qq, kk, v, page, split_size=256).view(hq, dh)
        want = v[far].bfloat16().float().repeat_interleave(hq // hkv, dim=0)
        assert (got - want).abs().max().item() < 2e-2, f"key {far}"


@pytest.mark.parametrize("window", [1, 5, 16, 17, 64, 100])
def test_attention_decode_window(window):
    torch.manual_seed(0)
    hq, hkv, dh, page, S = 4, 2, 64, 8, 230
    q = torch.randn(1, hq, dh).bfloat16().float()
    k = (torch.randn(S, hkv, dh) * 0.3).bfloat16().float()
    v = torch.randn(S, hkv, dh).bfloat16().float()
    torch.testing.assert_close(_decode(q, k, v, page, window=window, split_size=64), _windowed_plain(q, k, v, window), rtol=2 ** -7, atol=2 ** -7)
    # the key just outside the window matches the query and must stay unseen
    direction = torch.ones(dh) / math.sqrt(dh)
    qq = (direction * 40).expand(1, hq, dh).clone()
    kk = k.clone()
    kk[S - 1 - window] = direction * 10
    got = _decode(qq, kk, v, page, window=window, split_size=64)
    torch.testing.assert_close(got, _windowed_plain(qq, kk.bfloat16().float(), v, window), rtol=2 ** -6, atol=2 ** -6)
    # pages before the window are released (-1 in the block table) and must not be touched
    k_pages, v_pages, table = _paged(k.bfloat16(), v.bfloat16(), page, 40, dtype=torch.bfloat16)
    first_needed = (S - window) // page
    table = [-1 if blk < first_needed else pg for blk, pg in enumerate(table)]
    out = _ops().attention_decode(
        q.reshape(1, hq * dh).bfloat16().to(DEV), hq, hkv, dh, k_pages, v_pages, _i32([0]), _i32([S - 1]), _i32([table]), window, dh ** -0.5, window + 15
    )
    torch.testing.assert_close(out.float().cpu(), _windowed_plain(q, k, v, window), rtol=2 ** -7, atol=2 ** -7)


def test_attention_decode_batch_with_different_lengths():
    torch.manual_seed(0)
    hq, hkv, dh, page = 32, 8, 128, 16
    lens = [1, 700, 64, 33, 2500, 250]
    n_pages = sum(-(-n // page) for n in lens) + 5
    k_pages = torch.full((n_pages, hkv, page, dh), 30.0, dtype=torch.bfloat16)
    v_pages = torch.full((n_pages, hkv, page, dh), -30.0, dtype=torch.bfloat16)
    free = torch.randperm(n_pages).tolist()
    tables, wants, qs = [], [], []
    for S in lens:
        k, v, q = torch.randn(S, hkv, dh).bfloat16(), torch.randn(S, hkv, dh).bfloat16(), torch.randn(1, hq, dh).bfloat16()
        table = [free.pop() for _ in range(-(-S // page))]
        for pos in range(S):
            k_pages[table[pos // page], :, pos % page] = k[pos]
            v_pages[table[pos // page], :, pos % page] = v[pos]
        tables.append(table + [-1] * (160 - len(table)))
        wants.append(plain.attention(q.float(), k.float(), v.float()))
        qs.append(q.reshape(1, hq * dh))
    # queries sit in a wider row, as in the fused q|k|v buffer
    wide = torch.cat([torch.cat(qs), torch.randn(len(lens), 2 * hkv * dh).bfloat16()], dim=1).to(DEV)
    # the launch's splits: planned for equal lengths, planned for unequal ones, and given
    for split, uneven in ((None, False), (None, True), (64, False), (512, False)):
        out = _ops().attention_decode(
            wide, hq, hkv, dh, k_pages.to(DEV), v_pages.to(DEV), _i32(list(range(len(lens)))), _i32([n - 1 for n in lens]),
            _i32(tables), 0, dh ** -0.5, max(lens), split_size=split, uneven=uneven,
        )
        torch.testing.assert_close(out.float().cpu(), torch.cat(wants), rtol=2 ** -7, atol=2 ** -7)


def _fill_pages(k_pages, v_pages, table, k, v):
    """Write dense keys/values [S, Hkv, dh] into the pages ``table`` names, whole pages at a time."""
    S, hkv, dh = k.shape
    page = k_pages.shape[2]
    blocks = -(-S // page)
    pad = blocks * page - S
    idx = torch.tensor(table[:blocks])
    for pages, x in ((k_pages, k), (v_pages, v)):
        if pad:
            x = torch.cat([x, pages[idx[-1], :, page - pad :].transpose(0, 1).to(x.dtype)])
        pages[idx] = x.view(blocks, page, hkv, dh).transpose(1, 2).to(pages.dtype)


@pytest.mark.parametrize("batch, S", [(1, 32768), (8, 32768), (64, 8192)])
def test_attention_decode_at_the_longest_contexts_that_are_measured(batch, S):
    """32,768 keys for one request and for eight (32 splits of 1,024 keys), and 64 requests of 8,192 (8 splits;
    and unsplit, one block walking all keys of a request, no merge): the launches of the context sweep and of
    the batch-64 measurement.  Random scores in most rows; in some a single key, near
    the start, at a split's edge or at the end, that outweighs all others."""
    ops = _ops()
    hq, hkv, dh, page = 32, 8, 128, 16
    assert ops.plan_decode_splits(batch, hkv, S) == {1: (1024, 32), 8: (1024, 32), 64: (1024, 8)}[batch]
    g = torch.Generator().manual_seed(batch)
    lens = [S - (0, 1, 15, 16, 17, 700, 0, 63)[i % 8] for i in range(batch)]
    sharp = {0: 4095 if batch > 1 else None, 1: 0, 2: 4096, 3: lens[3 % batch] - 1, 5: 1023, 6: 1024, 7: S // 2 + 17}
    n_pages = sum(-(-n // page) for n in lens) + 5
    k_pages = torch.full((n_pages, hkv, page, dh), 30.0, dtype=torch.bfloat16)
    v_pages = torch.full((n_pages, hkv, page, dh), -30.0, dtype=torch.bfloat16)
    free = torch.randperm(n_pages, generator=g).tolist()
    tables, wants, qs = [], [], []
    width = -(-S // page)
    for i, n in enumerate(lens):
        k = torch.randn(n, hkv, dh, generator=g).bfloat16()
        v = torch.randn(n, hkv, dh, generator=g).bfloat16()
        q = (torch.randn(1, hq, dh, generator=g) * 2).bfloat16()
        far = sharp.get(i) if i < 8 else None
        if far is not None:
            direction = torch.randn(dh, generator=g)
            direction /= direction.norm()
            k[far] = (direction * 12).bfloat16()
            q = (direction * 12 * math.sqrt(dh) / 3).expand(1, hq, dh).bfloat16()
        table = [free.pop() for _ in range(-(-n // page))]
        _fill_pages(k_pages, v_pages, table, k, v)
        tables.append(table + [-1] * (width - len(table)))
        wants.append(plain.attention(q.float().to(DEV), k.float().to(DEV), v.float().to(DEV)).cpu())
        if far is not None:  # the one key's value, to a part in a thousand
            assert (wants[-1].view(hq, dh) - v[far].float().repeat_interleave(hq // hkv, dim=0)).abs().max() < 0.05
        qs.append(q.reshape(1, hq * dh))
    out = ops.attention_decode(
        torch.cat(qs).to(DEV), hq, hkv, dh, k_pages.to(DEV), v_pages.to(DEV), _i32(list(range(batch))), _i32([n - 1 for n in lens]),
        _i32(tables), 0, dh ** -0.5, max(lens),
    )
    torch.testing.assert_close(out.float().cpu(), torch.cat(wants), rtol=2 ** -7, atol=2 ** -7)
    if batch == 64:  # and without splits
        whole = ops.attention_decode(
            torch.cat(qs).to(DEV), hq, hkv, dh, k_pages.to(DEV), v_pages.to(DEV), _i32(list(range(batch))), _i32([n - 1 for n in lens]),
            _i32(tables), 0, dh ** -0.5, max(lens), split_size=S,
        )
        torch.testing.assert_close(whole.float().cpu(), torch.cat(wants), rtol=2 ** -7, atol=2 ** -7)
    if batch == 1:  # the one request again, with one key that outweighs the others, in turn at these places
        k_dev, v_dev = k_pages.to(DEV), v_pages.to(DEV)
        for far in (0, 1023, 1024, 20000, S - 65, S - 1):
            direction = torch.randn(dh, generator=g)
            direction /= direction.norm()
            kept = k_dev[table[far // page], :, far % page].clone()
            k_dev[table[far // page], :, far % page] = (direction * 12).bfloat16().to(DEV)
            qq = (direction * 12 * math.sqrt(dh) / 3).expand(1, hq, dh).reshape(1, hq * dh).bfloat16().to(DEV)
            got = ops.attention_decode(qq, hq, hkv, dh, k_dev, v_dev, _i32([0]), _i32([S - 1]), _i32(tables), 0, dh ** -0.5, S)
            k_dev[table[far // page], :, far % page] = kept
            err = (got.float().cpu().view(hq, dh) - v[far].float().repeat_interleave(hq // hkv, dim=0)).abs().max().item()
            assert err < 3e-2, f"key {far}: {err}"


def test_attention_decode_says_what_it_takes():
    ops = _ops()
    assert ops.decode_attention_supported(torch.bfloat16, 32, 8, 128)
    assert not ops.decode_attention_supported(torch.float32, 32, 8, 128)
    assert not ops.decode_attention_supported(torch.bfloat16, 6, 3, 48)
    assert not ops.decode_attention_supported(torch.bfloat16, 16, 1, 256)
    assert ops.plan_decode_splits(8, 8, 8192) == (1024, 8)
    assert ops.plan_decode_splits(64, 8, 8192) == (1024, 8) and ops.plan_decode_splits(64, 8, 4095) == (4095 + 1, 1)
    assert ops.plan_decode_splits(64, 8, 8192, uneven=True) == (512, 16)
    assert ops.plan_decode_splits(2, 8, 8192, uneven=True) == (512, 16)
    assert ops.plan_decode_splits(6, 8, 4096) == (448, 10) and ops.plan_decode_splits(6, 8, 4096, uneven=True) == (448, 10)  # what equal requests get is shorter still
    assert ops.plan_decode_splits(2, 8, 4096) == (256, 16)
    assert ops.plan_decode_splits(64, 8, 40) == (128, 1)
    assert ops.plan_decode_splits(1, 8, 8192) == (256, 32) and ops.plan_decode_splits(1, 8, 2176) == (128, 17)


# ----------------------------------------------------------------------------- weight-streaming matrix product (decode)
@pytest.mark.parametrize(
    "m, n, k",
    [(1, 4096, 4096), (8, 6144, 4096), (8, 4096, 14336), (16, 1000, 256), (16, 300, 96), (9, 257, 688), (13, 2048, 1024),
     (3, 16, 8), (5, 31, 136), (4, 40, 128), (16, 128256 // 8, 512)],
)
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_gemm_stream(m, n, k, out_dtype):
    """The coalesced-fetch kernel: every row count's fetch groups, K with and without a partial
    step, N that is no multiple of 16, every split of K."""
    torch.manual_seed(0)
    x = torch.randn(m, k).bfloat16()
    w = (torch.randn(n, k) * 0.05).bfloat16()
    want = x.double() @ w.double().T
    tol = (1e-4 if out_dtype == torch.float32 else 2 ** -8) * want.abs().max().item() + 1e-5
    for waves in (0, 1, 2, 4, 8):
        got = _ops().gemm_stream(x.to(DEV), w.to(DEV), out_dtype, waves=waves).float().cpu()
        assert (got.double() - want).abs().max().item() <= tol, f"waves={waves}"


@pytest.mark.parametrize("m, f, k", [(1, 4096, 1024), (8, 14336, 4096), (5, 100, 136), (16, 688, 96), (12, 24, 8), (3, 13, 264)])
def test_gemm_stream_glu_equals_the_product_followed_by_the_gate(m, f, k):
    """The same roundings as the two kernels it replaces; the 32-bit sums may differ in their last
    bit (blocks walk K from different starting steps), so single results may move by one rounding."""
    torch.manual_seed(1)
    x = torch.randn(m, k).bfloat16().to(DEV)
    w = (torch.randn(2 * f, k) * 0.1).bfloat16().to(DEV)
    for waves in (0, 1, 2, 4, 8):
        want = _ops().silu_mul(_ops().gemm_stream(x, w, torch.bfloat16, waves=waves))
        for cols in (16, 8):  # both shapes of a block: gate and up tiles of 16 columns, or 8 + 8 rows in one tile
            got = _ops().gemm_stream_glu(x, w, waves=waves, cols=cols)
            torch.testing.assert_close(got.float(), want.float(), rtol=2 ** -6, atol=2 ** -8 * want.float().abs().max().item(), msg=f"waves={waves} cols={cols}")
            assert (got != want).float().mean().item() < 0.05, f"waves={waves} cols={cols}"
    ref = torch.nn.functional.silu(x.float() @ w[:f].float().T) * (x.float() @ w[f:].float().T)
    torch.testing.assert_close(_ops().linear_glu(x, w).float(), ref, rtol=2 ** -6, atol=2 ** -6 * ref.abs().max().item())


def _pieces_of_squares(rows: torch.Tensor, n_pieces: int) -> torch.Tensor:
    """float32 [n_pieces, 16] whose columns add up to each row's sum of squares: the squares of the
    elements dealt out to the pieces in turn; the columns past the last row hold rubbish."""
    sq = rows.float() ** 2
    pad = (-sq.shape[1]) % n_pieces
    sq = torch.nn.functional.pad(sq, (0, pad))
    out = torch.full((n_pieces, 16), float("nan"), device=rows.device)
    out[:, : rows.shape[0]] = sq.reshape(sq.shape[0], -1, n_pieces).sum(1).T
    return out


@pytest.mark.parametrize("m, n, k", [(1, 4096, 4096), (8, 4096, 14336), (16, 300, 96), (9, 260, 688), (13, 2048, 1024), (3, 16, 8),
                                     (5, 36, 136), (4, 2052, 128)])
def test_gemm_stream_residual_adds_the_product_to_its_rows_and_leaves_their_sums_of_squares(m, n, k):
    """The sum is the one the norm kernel would have formed from the stored product (product rounded,
    added in 32-bit, rounded), bit for bit; beside it the same rows times the gain, and the squares
    of the stored rows by 16 columns."""
    torch.manual_seed(4)
    x = torch.randn(m, k).bfloat16().to(DEV)
    w = (torch.randn(n, k) * k ** -0.5).bfloat16().to(DEV)
    h = (torch.randn(m, n) * torch.logspace(-1, 1, m)[:, None]).bfloat16().to(DEV)
    gain = (0.3 + 2 * torch.rand(n)).bfloat16().to(DEV)
    for waves in (0, 1, 2, 4, 8):
        got, gained, sums = _ops().gemm_stream_residual(x, w, h, gain, waves=waves)
        want = (h.float() + _ops().gemm_stream(x, w, torch.bfloat16, waves=waves).float()).bfloat16()
        assert torch.equal(got, want), f"waves={waves}"
        assert torch.equal(gained, (want.float() * gain.float()).bfloat16()), f"waves={waves}"
        sq = torch.nn.functional.pad(want.float() ** 2, (0, (-n) % 16)).reshape(m, -1, 16).sum(-1)
        assert sums.shape == (sq.shape[1], 16)
        torch.testing.assert_close(sums[:, :m].T, sq, rtol=1e-5, atol=1e-30, msg=f"waves={waves}")
    pending = _ops().PendingProduct(x, w, 0)
    assert pending.shape == (m, n) and torch.equal(_ops().resolved(pending), _ops().gemm_stream(x, w))
    rows, normed = pending.added_to(h, gain, 1e-3)
    assert torch.equal(rows, want) and normed.rows is rows and normed.shape == (m, n)
    # what the statistics stand for is the norm kernel's result on the new rows
    assert torch.equal(_ops().resolved(normed), _ops().rmsnorm(want, gain, 1e-3))


def test_gemm_stream_residual_says_its_limits():
    from torchllms_amd.kernels.lib import KernelError

    def z(*shape):
        return torch.zeros(*shape, dtype=torch.bfloat16, device=DEV)

    x = z(2, 64)
    with pytest.raises(KernelError, match="multiple of 4"):
        _ops().gemm_stream_residual(x, z(30, 64), z(2, 30), z(30))
    with pytest.raises(KernelError, match="rows to add to"):
        _ops().gemm_stream_residual(x, z(32, 64), z(3, 32), z(32))
    with pytest.raises(KernelError, match="a gain of shape"):
        _ops().gemm_stream_residual(x, z(32, 64), z(2, 32), z(31))
    # the statistics must be those of the rows that are multiplied
    norm = _ops().NormedRows(x, x.clone(), torch.ones(4, 16, device=DEV), 1e-5, z(64))
    with pytest.raises(KernelError, match="do not belong"):
        _ops().gemm_stream_glu(x, z(32, 64), norm=norm)


@pytest.mark.parametrize("m, f, k, pieces", [(1, 4096, 1024, 64), (8, 1024, 4096, 256), (5, 100, 136, 9), (16, 688, 96, 6), (12, 24, 8, 1),
                                             (3, 13, 264, 33), (16, 64, 2048, 300)])
def test_gemm_stream_glu_applies_a_norm_from_the_rows_sums_of_squares(m, f, k, pieces):
    """Rows of very different sizes, so another row's factor shows; an eps that counts for the small
    rows; any number of pieces, more than the lanes of a row hold ahead included."""
    torch.manual_seed(5)
    eps = 1e-2
    x = (torch.randn(m, k) * torch.logspace(-1.5, 1.5, m)[:, None]).bfloat16().to(DEV)
    w = (torch.randn(2 * f, k) * k ** -0.5).bfloat16().to(DEV)
    gain = (0.3 + 2 * torch.rand(k)).bfloat16().to(DEV)
    norm = _ops().NormedRows(x, (x.float() * gain.float()).bfloat16(), _pieces_of_squares(x, pieces), eps, gain)
    xn = x.float() * torch.rsqrt((x.float() ** 2).mean(-1, keepdim=True) + eps) * gain.float()
    ref = torch.nn.functional.silu(xn @ w[:f].float().T) * (xn @ w[f:].float().T)
    tol = dict(rtol=2 ** -6, atol=2 ** -6 * ref.abs().max().item())
    torch.testing.assert_close(_ops().resolved(norm).float(), xn, rtol=2 ** -6, atol=1e-6)
    for waves in (0, 1, 2, 4, 8):
        for cols in (16, 8):
            got = _ops().gemm_stream_glu(norm.gained, w, waves=waves, cols=cols, norm=norm)
            torch.testing.assert_close(got.float(), ref, **tol, msg=f"waves={waves} cols={cols}")
    torch.testing.assert_close(_ops().linear_glu(norm, w).float(), ref, **tol)


def test_normed_rows_are_normed_first_where_another_kernel_serves_the_shape():
    """``linear_glu`` and ``qkv_rope_store`` given ``NormedRows`` for a matrix that the table sends to the
    library: the norm kernel runs on the rows, then whatever serves the shape."""
    from torchllms_amd.kernels import products

    torch.manual_seed(8)
    m, k, f, eps = 5, 64, 48, 1e-3
    x = torch.randn(m, k).bfloat16().to(DEV)
    gain = (0.5 + torch.rand(k)).bfloat16().to(DEV)
    w = (torch.randn(2 * f, k) * k ** -0.5).bfloat16().to(DEV)
    norm = _ops().NormedRows(x, (x.float() * gain.float()).bfloat16(), _pieces_of_squares(x, 4), eps, gain)
    keys = [(2 * f, k, products.row_bucket(m), use) for use in ("glu", "qkv")]
    saved = {key: products.LINEAR_CHOICE.get(key) for key in keys}
    try:
        for key in keys:
            products.LINEAR_CHOICE[key] = None
        y = _ops().rmsnorm(x, gain, eps)
        assert torch.equal(_ops().linear_glu(norm, w), _ops().silu_mul(torch.nn.functional.linear(y, w)))
        pos = _i32(list(range(m)))
        inv_freq = plain.rope_inverse_frequencies(16, 10000.0, None).to(DEV)
        table = _ops().rope_table(pos, inv_freq)
        got = _ops().qkv_rope_store(norm, w, None, 2, 2, 16, pos, inv_freq, 16, 0, table, None, None, None, 0)
        want = _ops().qkv_rope_store(y, w, None, 2, 2, 16, pos, inv_freq, 16, 0, table, None, None, None, 0)
        assert torch.equal(got, want)
    finally:
        for key, choice in saved.items():
            if choice is None:
                products.LINEAR_CHOICE.pop(key, None)
            else:
                products.LINEAR_CHOICE[key] = choice


@pytest.mark.parametrize("m, hq, hkv, dh, rot, page, k, pieces", [(8, 32, 8, 128, 128, 16, 4096, 256), (1, 4, 4, 64, 64, 16, 256, 16),
                                                                   (13, 6, 3, 48, 24, 4, 136, 9), (16, 5, 1, 20, 0, 8, 64, 40), (3, 2, 2, 16, 16, 2, 8, 1)])
def test_gemm_stream_qkv_applies_a_norm_from_the_rows_sums_of_squares(m, hq, hkv, dh, rot, page, k, pieces):
    """Against the norm kernel followed by the fused projection: queries, and keys and values in their pages."""
    torch.manual_seed(6)
    eps = 1e-3
    width = (hq + 2 * hkv) * dh
    x = (torch.randn(m, k) * torch.logspace(-1.5, 1.5, m)[:, None]).bfloat16().to(DEV)
    w = (torch.randn(width, k) * k ** -0.5).bfloat16().to(DEV)
    gain = (0.3 + 2 * torch.rand(k)).bfloat16().to(DEV)
    norm = _ops().NormedRows(x, (x.float() * gain.float()).bfloat16(), _pieces_of_squares(x, pieces), eps, gain)
    pos = torch.randint(0, 9000, (m,))
    inv_freq = plain.rope_inverse_frequencies(rot, 500000.0, None).to(DEV) if rot else None
    table = _ops().rope_table(_i32(pos.tolist()), inv_freq) if rot else None
    n_pages = 40
    sm = _i32(torch.randperm(n_pages * page)[:m].tolist())
    ka, va = _pages(n_pages, hkv, page, dh, torch.bfloat16)
    qa = _ops().gemm_stream_qkv(_ops().rmsnorm(x, gain, eps), w, hq, hkv, dh, rot, table, ka, va, sm, page)
    for waves in (0, 1, 2, 4, 8):
        kb, vb = _pages(n_pages, hkv, page, dh, torch.bfloat16)
        qb = _ops().gemm_stream_qkv(norm.gained, w, hq, hkv, dh, rot, table, kb, vb, sm, page, waves=waves, norm=norm)
        tol = dict(rtol=2 ** -6, atol=2 ** -7 * qa[:, : hq * dh].float().abs().max().item())
        torch.testing.assert_close(qb[:, : hq * dh].float(), qa[:, : hq * dh].float(), **tol, msg=f"waves={waves}")
        torch.testing.assert_close(kb.float(), ka.float(), **tol)
        torch.testing.assert_close(vb.float(), va.float(), **tol)
    kc, vc = _pages(n_pages, hkv, page, dh, torch.bfloat16)
    qc = _ops().qkv_rope_store(norm, w, None, hq, hkv, dh, _i32(pos.tolist()), inv_freq, rot, 0, table, kc, vc, sm, page)
    torch.testing.assert_close(qc[:, : hq * dh].float(), qa[:, : hq * dh].float(), **tol)
    torch.testing.assert_close(kc.float(), ka.float(), **tol)


def test_gemm_stream_takes_strided_rows_and_says_its_limits():
    from torchllms_amd.kernels.lib import KernelError

    torch.manual_seed(0)
    wide = torch.randn(6, 512).bfloat16().to(DEV)
    x = wide[:, :256]  # row stride 512
    w = torch.randn(40, 256).bfloat16().to(DEV)
    got = _ops().gemm_stream(x, w).float().cpu()
    torch.testing.assert_close(got, (x.float() @ w.float().T).cpu(), rtol=2 ** -7, atol=0.1)
    with pytest.raises(KernelError, match="exceeds 16"):
        _ops().gemm_stream(torch.zeros(17, 64, dtype=torch.bfloat16, device=DEV), w[:, :64].contiguous())
    with pytest.raises(KernelError, match="multiple of 8"):
        _ops().gemm_stream(torch.zeros(2, 12, dtype=torch.bfloat16, device=DEV), torch.zeros(4, 12, dtype=torch.bfloat16, device=DEV))


def test_linear_sends_what_the_streaming_kernel_does_not_take_to_the_library():
    torch.manual_seed(0)
    wide = torch.randn(6, 512).bfloat16().to(DEV)
    x = wide[:, :256]  # row stride 512
    w = torch.randn(40, 256).bfloat16().to(DEV)
    got = _ops().linear(x, w).float().cpu()
    torch.testing.assert_close(got, (x.float() @ w.float().T).cpu(), rtol=2 ** -7, atol=0.1)
    odd = _ops().linear(torch.ones(2, 12, dtype=torch.bfloat16, device=DEV), torch.ones(4, 12, dtype=torch.bfloat16, device=DEV))
    assert odd.float().cpu().tolist() == [[12.0] * 4] * 2
    big = _ops().linear(torch.ones(70, 16, dtype=torch.bfloat16, device=DEV), torch.ones(4, 16, dtype=torch.bfloat16, device=DEV), out_dtype=torch.float32)
    assert big.dtype == torch.float32 and big.shape == (70, 4)
    assert big.cpu().tolist() == [[16.0] * 4] * 70


def test_tune_linear_remembers_a_choice_for_every_row_bucket():
    ops = _ops()
    torch.manual_seed(0)
    weights = [torch.randn(48, 64, device=DEV).bfloat16() for _ in range(2)]
    for key in [k for k in products.LINEAR_CHOICE if k[:2] == (48, 64)]:
        del products.LINEAR_CHOICE[key]
    ops.tune_linear(weights)
    ops.tune_linear(weights, use="glu")
    for bucket in ops.ROW_BUCKETS:
        if bucket <= ops.STREAM_MAX_ROWS:
            assert products.LINEAR_CHOICE[(48, 64, bucket, "plain")] in (None,) + tuple(("stream", w) for w in ops.STREAM_WAVE_CHOICES)
            assert products.LINEAR_CHOICE[(48, 64, bucket, "glu")] in (None,) + tuple(("stream", w, c) for w in ops.STREAM_WAVE_CHOICES for c in (8, 16))
        else:
            assert products.LINEAR_CHOICE[(48, 64, bucket, "plain")] is None  # K = 64 is no multiple of 128: the library
    x = torch.randn(5, 64, device=DEV).bfloat16()
    got = ops.linear(x, weights[0]).float().cpu()
    torch.testing.assert_close(got, (x.float() @ weights[0].float().T).cpu(), rtol=2 ** -7, atol=0.1)
    glu = (torch.nn.functional.silu(x.float() @ weights[0][:24].float().T) * (x.float() @ weights[0][24:].float().T)).cpu()
    torch.testing.assert_close(ops.linear_glu(x, weights[0]).float().cpu(), glu, rtol=2 ** -6, atol=0.1)


# ----------------------------------------------------------------------------- shared-activation matrix product (17 to 128 rows)
@pytest.mark.parametrize(
    "m, n, k",
    [(64, 4096, 4096), (32, 6144, 4096), (17, 200, 128), (64, 4100, 384), (33, 72, 2048), (48, 1000, 1024), (5, 64, 256),
     (64, 128, 14336), (49, 130, 640), (128, 4096, 4096), (65, 200, 384), (100, 1000, 1024), (127, 72, 2048)],
)
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_gemm_wide(m, n, k, out_dtype):
    """All row tiles (32, 64 and 128), N that is no multiple of a block's columns, one step of K and
    many, every block shape, splits of K that divide the steps and that do not, both buffer counts
    (three buffers of the largest tile with two strips do not fit LDS and are refused)."""
    from torchllms_amd.kernels.lib import KernelError

    torch.manual_seed(0)
    x = torch.randn(m, k).bfloat16()
    w = (torch.randn(n, k) * 0.05).bfloat16()
    want = x.double() @ w.double().T
    tol = (1e-4 if out_dtype == torch.float32 else 2 ** -8) * want.abs().max().item() + 1e-5
    for strips in (1, 2):
        for splits in (1, 2, 3, 8):
            for stages in (2, 3):
                if not _ops().wide_fits(m, strips, stages):
                    with pytest.raises(KernelError, match="do not fit into LDS"):
                        _ops().gemm_wide(x.to(DEV), w.to(DEV), out_dtype, strips, splits, stages)
                    continue
                got = _ops().gemm_wide(x.to(DEV), w.to(DEV), out_dtype, strips, splits, stages).float().cpu()
                assert (got.double() - want).abs().max().item() <= tol, f"strips={strips} splits={splits} stages={stages}"


@pytest.mark.parametrize("m, f, k", [(64, 14336, 4096), (32, 1000, 256), (17, 40, 128), (50, 72, 1152), (128, 4096, 2048), (77, 200, 384)])
def test_gemm_wide_glu_equals_the_product_followed_by_the_gate(m, f, k):
    """The same roundings as the two kernels it replaces (see the streaming kernel's test)."""
    torch.manual_seed(1)
    x = torch.randn(m, k).bfloat16().to(DEV)
    w = (torch.randn(2 * f, k) * 0.1).bfloat16().to(DEV)
    ref = torch.nn.functional.silu(x.float() @ w[:f].float().T) * (x.float() @ w[f:].float().T)
    for strips in (1, 2):
        for stages in (2, 3):
            if not _ops().wide_fits(m, strips, stages):
                continue
            want = _ops().silu_mul(_ops().gemm_wide(x, w, torch.bfloat16, strips, 1, stages))
            got = _ops().gemm_wide_glu(x, w, strips, stages)
            torch.testing.assert_close(got.float(), want.float(), rtol=2 ** -6, atol=2 ** -8 * want.float().abs().max().item(), msg=f"strips={strips}")
            assert (got != want).float().mean().item() < 0.05, f"strips={strips} stages={stages}"
            torch.testing.assert_close(got.float(), ref, rtol=2 ** -6, atol=2 ** -6 * ref.abs().max().item())


@pytest.mark.parametrize("m, hq, hkv, dh, rot, page, k", [(64, 32, 8, 128, 128, 16, 4096), (32, 4, 4, 64, 64, 16, 256),
                                                           (23, 6, 3, 48, 24, 4, 384), (40, 5, 1, 20, 0, 8, 128),
                                                           (128, 8, 2, 64, 64, 16, 1024), (90, 6, 3, 48, 24, 4, 384)])
@pytest.mark.parametrize("with_pages", [True, False])
def test_gemm_wide_qkv_equals_product_then_rotary_kernel(m, hq, hkv, dh, rot, page, k, with_pages):
    """The split product whose second kernel rotates and scatters, against product and rotary
    kernel in turn, on every output; a row whose slot is negative stores nothing."""
    torch.manual_seed(2)
    width = (hq + 2 * hkv) * dh
    x = torch.randn(m, k).bfloat16().to(DEV)
    w = (torch.randn(width, k) * k ** -0.5).bfloat16().to(DEV)
    pos = torch.randint(0, 9000, (m,))
    inv_freq = plain.rope_inverse_frequencies(rot, 500000.0, None).to(DEV) if rot else None
    table = _ops().rope_table(_i32(pos.tolist()), inv_freq) if rot else None
    n_pages = 160
    slots = torch.randperm(n_pages * page)[:m].tolist()
    slots[1] = -1
    sm = _i32(slots) if with_pages else None
    ka, va = _pages(n_pages, hkv, page, dh, torch.bfloat16) if with_pages else (None, None)
    qa = _ops().gemm_wide(x, w, torch.bfloat16, 1, 1, 2)
    _ops().rope_kv_write(qa, hq, hkv, dh, _i32(pos.tolist()), inv_freq, rot, 0, ka, va, sm, page if with_pages else 0, cos_sin=table)
    cols = hq * dh if with_pages else width  # with pages only the queries of the buffer are defined
    tol = dict(rtol=2 ** -7, atol=2 ** -8 * qa.float().abs().max().item())
    for strips, splits, stages in ((1, 1, 3), (1, 2, 3), (2, 4, 2), (1, 8, 3)):
        kb, vb = _pages(n_pages, hkv, page, dh, torch.bfloat16) if with_pages else (None, None)
        qb = _ops().gemm_wide_qkv(x, w, hq, hkv, dh, rot, table, kb, vb, sm, page if with_pages else 0, strips, splits, stages)
        torch.testing.assert_close(qb[:, :cols].float(), qa[:, :cols].float(), **tol)
        assert (qb[:, :cols] != qa[:, :cols]).float().mean().item() < 0.05  # only last-bit differences of the sums
        if with_pages:
            torch.testing.assert_close(kb.float(), ka.float(), **tol)
            torch.testing.assert_close(vb.float(), va.float(), **tol)
            assert (kb.float().abs().sum(dim=(1, 3)) > 0).sum().item() == m - 1  # one slot per stored row


def test_gemm_wide_takes_strided_rows_and_says_its_limits():
    from torchllms_amd.kernels.lib import KernelError

    torch.manual_seed(0)
    buf = torch.randn(40, 512).bfloat16().to(DEV)
    x = buf[:, :256]  # row stride 512
    w = torch.randn(70, 256).bfloat16().to(DEV)
    got = _ops().gemm_wide(x, w, torch.float32, 2, 2).cpu()
    torch.testing.assert_close(got, (x.float() @ w.float().T).cpu(), rtol=1e-4, atol=1e-3)
    with pytest.raises(KernelError, match="exceeds 128"):
        _ops().gemm_wide(torch.zeros(129, 256, dtype=torch.bfloat16, device=DEV), w)
    with pytest.raises(KernelError, match="multiple of 128"):
        _ops().gemm_wide(torch.zeros(20, 64, dtype=torch.bfloat16, device=DEV), w[:, :64].contiguous())
    with pytest.raises(KernelError, match="stages"):
        _ops().gemm_wide(x, w, torch.float32, 1, 1, 4)


@pytest.mark.parametrize("m, n, k, splits", [(64, 4096, 1024, 4), (20, 2048, 512, 8), (33, 72, 384, 2), (17, 8192, 256, 3), (18, 264, 128, 1),
                                           (19, 520, 1408, 11)])
@pytest.mark.parametrize("weight_dtype", [torch.bfloat16, torch.float32])
def test_rmsnorm_adds_up_a_split_product_as_the_reduce_kernel_would(m, n, k, splits, weight_dtype):
    """A product left as the sums of its splits, taken as the delta of the norm: bit for bit what
    the product's own second kernel followed by the norm gives (same order of additions, same
    roundings), for the whole batch, with the sum returned, and for gathered rows."""
    ops = _ops()
    torch.manual_seed(5)
    x = torch.randn(m, k).bfloat16().to(DEV)
    w = (torch.randn(n, k) * 0.05).bfloat16().to(DEV)
    h = torch.randn(m, n).bfloat16().to(DEV)
    g = (1 + 0.1 * torch.randn(n)).to(weight_dtype).to(DEV)
    whole = ops.gemm_wide(x, w, torch.bfloat16, 1, splits, 3)
    left = ops.gemm_wide(x, w, torch.bfloat16, 1, splits, 3, leave_split=True)
    assert isinstance(left, ops.SplitSums) and left.shape == (m, n) and left.partial.shape[0] == min(splits, k // 128)
    assert torch.equal(left.resolve(), whole)
    want_h, want_y = ops.rmsnorm(h, g, 1e-5, delta=whole, return_sum=True)
    got_h, got_y = ops.rmsnorm(h, g, 1e-5, delta=left, return_sum=True)
    assert torch.equal(got_h, want_h) and torch.equal(got_y, want_y)
    rows = _i32([m - 1, 0, 3, 3])
    assert torch.equal(ops.rmsnorm(h, g, 1e-5, delta=left, rows=rows), ops.rmsnorm(h, g, 1e-5, delta=whole, rows=rows))
    # against the formula
    ref = plain.rms_norm((h.float() + whole.float()).bfloat16().float().cpu(), g.float().cpu(), 1e-5)
    torch.testing.assert_close(got_y.float().cpu(), ref, rtol=2 ** -6, atol=2 ** -6)


def test_rmsnorm_adds_the_splits_first_where_its_kernel_does_not_take_the_width():
    ops = _ops()
    torch.manual_seed(6)
    x = torch.randn(24, 256).bfloat16().to(DEV)
    w = (torch.randn(100, 256) * 0.05).bfloat16().to(DEV)  # 100 columns: no multiple of 8
    h = torch.randn(24, 100).bfloat16().to(DEV)
    g = torch.ones(100, dtype=torch.bfloat16, device=DEV)
    left = ops.gemm_wide(x, w, torch.bfloat16, 1, 2, 2, leave_split=True)
    want = ops.rmsnorm(h, g, 1e-6, delta=ops.gemm_wide(x, w, torch.bfloat16, 1, 2, 2))
    assert torch.equal(ops.rmsnorm(h, g, 1e-6, delta=left), want)


def test_linear_to_sum_leaves_a_product_split_only_where_it_was_tuned_to_be_split():
    ops = _ops()
    torch.manual_seed(7)
    w = (torch.randn(96, 512, device=DEV) * 0.05).bfloat16()
    x = torch.randn(40, 512, device=DEV).bfloat16()
    want = (x.float() @ w.float().T).cpu()
    key = (96, 512, 64, "sum")
    saved = products.LINEAR_CHOICE.get(key, "absent")
    try:
        for choice, split in ((None, False), (("wide", 1, 1, 3), False), (("wide", 1, 4, 3), True), (("wide", 2, 2, 2), True)):
            products.LINEAR_CHOICE[key] = choice
            got = ops.linear_to_sum(x, w)
            assert isinstance(got, ops.SplitSums) == split, choice
            if split:
                got = got.resolve()
            torch.testing.assert_close(got.float().cpu(), want, rtol=2 ** -7, atol=0.05)
        small = ops.linear_to_sum(x[:3], w)  # few rows: the streaming kernel, which adds its splits inside the block
        assert isinstance(small, torch.Tensor)
        f32 = ops.linear_to_sum(x.float(), w.float())
        assert isinstance(f32, torch.Tensor) and f32.dtype == torch.float32
    finally:
        if saved == "absent":
            products.LINEAR_CHOICE.pop(key, None)
        else:
            products.LINEAR_CHOICE[key] = saved


def test_tune_linear_measures_the_wide_kernel_from_17_rows_on():
    ops = _ops()
    torch.manual_seed(0)
    weights = [(torch.randn(96, 256, device=DEV) * 0.1).bfloat16() for _ in range(2)]
    for key in [k for k in products.LINEAR_CHOICE if k[:2] == (96, 256)]:
        del products.LINEAR_CHOICE[key]
    for use in ops.LINEAR_USES:
        ops.tune_linear(weights, use=use)
    allowed = {None} | {("wide",) + c for c in ops.WIDE_CHOICES if c[1] <= 2}
    for use in ops.LINEAR_USES:
        assert products.LINEAR_CHOICE[(96, 256, 32, use)] in allowed and products.LINEAR_CHOICE[(96, 256, 64, use)] in allowed
    # whatever was chosen, and each of the kernel's launches when it is forced, gives the product
    x = torch.randn(40, 256, device=DEV).bfloat16()
    want = (x.float() @ weights[0].float().T).cpu()
    torch.testing.assert_close(ops.linear(x, weights[0]).float().cpu(), want, rtol=2 ** -7, atol=0.05)
    glu_ref = (torch.nn.functional.silu(x.float() @ weights[0][:48].float().T) * (x.float() @ weights[0][48:].float().T)).cpu()
    for choice in sorted(allowed - {None}) + [("wide", 1, 2, 2)]:
        products.LINEAR_CHOICE[(96, 256, 64, "plain")] = products.LINEAR_CHOICE[(96, 256, 64, "glu")] = choice
        torch.testing.assert_close(ops.linear(x, weights[0]).float().cpu(), want, rtol=2 ** -7, atol=0.05)
        torch.testing.assert_close(ops.linear_glu(x, weights[0]).float().cpu(), glu_ref, rtol=2 ** -6, atol=0.05)
    for use in ops.LINEAR_USES:
        del products.LINEAR_CHOICE[(96, 256, 64, use)]


# ----------------------------------------------------------------------------- prefill attention (MFMA)
def _prefill(rows, hq, hkv, dh, page, window=0, seed=0, key_groups=1):
    """Run the prefill kernel on a batch: ``rows`` = [(tokens cached after the step, new queries)].
    Returns (got, want): outputs for all new tokens, row after row."""
    torch.manual_seed(seed)
    n_pages = sum(-(-S // page) for S, _ in rows) + 4
    k_pages = torch.full((n_pages, hkv, page, dh), 40.0, dtype=torch.bfloat16)
    v_pages = torch.full((n_pages, hkv, page, dh), -40.0, dtype=torch.bfloat16)
    free = torch.randperm(n_pages).tolist()
    width = max(-(-S // page) for S, _ in rows)
    tables, wants, qs, qo, kv = [], [], [], [0], []
    for S, sq in rows:
        k = (torch.randn(S, hkv, dh) * 0.5).bfloat16()
        v = torch.randn(S, hkv, dh).bfloat16()
        q = (torch.randn(sq, hq, dh) * 2).bfloat16()
        table = [free.pop() for _ in range(-(-S // page))]
        for pos in range(S):
            k_pages[table[pos // page], :, pos % page] = k[pos]
            v_pages[table[pos // page], :, pos % page] = v[pos]
        tables.append(table + [-1] * (width - len(table)))
        wants.append(_windowed_plain(q.float(), k.float(), v.float(), window) if window else plain.attention(q.float(), k.float(), v.float()))
        qs.append(q.reshape(sq, hq * dh))
        qo.append(qo[-1] + sq)
        kv.append(S)
    ops = _ops()
    n = qo[-1]
    wide = torch.cat([torch.cat(qs), torch.randn(n, 2 * hkv * dh).bfloat16()], dim=1).to(DEV)
    qpt = ops.prefill_queries_per_tile(hq, hkv, dh)
    trow, tq0 = ops.prefill_tiles(qo, 0, len(rows), qpt, kv, window)  # in the balanced order the engine uses
    out = torch.zeros(n, hq * dh, dtype=torch.bfloat16, device=DEV)
    ops.attention_prefill(wide, hq, hkv, dh, k_pages.to(DEV), v_pages.to(DEV), _i32(qo), _i32(kv), _i32(tables), _i32(trow), _i32(tq0),
                          window, dh ** -0.5, out, key_groups=key_groups)
    return out.float().cpu(), torch.cat(wants)


@pytest.mark.parametrize(
    "hq, hkv, dh, page, rows",
    [
        (32, 8, 128, 16, [(300, 300)]),
        (32, 8, 128, 16, [(77, 77), (500, 2), (130, 64), (33, 33)]),
        (8, 1, 32, 16, [(200, 200), (65, 3)]),
        (4, 4, 64, 8, [(150, 150)]),
        (6, 2, 64, 8, [(90, 31), (40, 40)]),
        (16, 1, 128, 32, [(129, 129)]),
        (4, 1, 256, 16, [(100, 100), (70, 5)]),
        (5, 5, 32, 16, [(61, 61)]),
        (3, 1, 256, 2, [(61, 61), (30, 7)]),
        (8, 2, 128, 4, [(150, 150), (99, 6)]),
        (5, 5, 32, 128, [(261, 261), (140, 3)]),
        (2, 2, 64, 16, [(1, 1), (2, 2), (17, 16)]),
    ],
)
@pytest.mark.parametrize("key_groups", [1, 2])
def test_attention_prefill(hq, hkv, dh, page, rows, key_groups):
    """``key_groups`` = 2: two sets of waves per block take every second tile of keys each and add
    up at the end; a row of fewer keys than two tiles leaves the second set without any."""
    got, want = _prefill(rows, hq, hkv, dh, page, key_groups=key_groups)
    torch.testing.assert_close(got, want, rtol=2 ** -6, atol=2 ** -6)


def test_attention_prefill_takes_pages_of_a_power_of_two_only():
    """Pages of 12 tokens are refused by the MFMA kernel with a clear error (and sent to the plain
    kernel by the dispatcher: tests/test_gpu_random_configs.py runs such page sizes end to end); so
    are pages shorter than the rows that a wave fetches with one instruction (512 / head size)."""
    ops = _ops()
    assert ops.prefill_attention_supported(torch.bfloat16, 4, 2, 64, 16) and not ops.prefill_attention_supported(torch.bfloat16, 4, 2, 64, 12)
    with pytest.raises(ops.KernelError, match="page_size 12 is no power of two"):
        _prefill([(61, 61)], 5, 5, 32, 12)
    assert ops.prefill_attention_supported(torch.bfloat16, 4, 2, 64, 8) and not ops.prefill_attention_supported(torch.bfloat16, 4, 2, 64, 4)
    assert ops.prefill_attention_supported(torch.bfloat16, 4, 2, 256, 2) and not ops.prefill_attention_supported(torch.bfloat16, 4, 2, 32, 8)
    with pytest.raises(ops.KernelError, match="pages of 4 tokens are shorter than the 8 rows"):
        _prefill([(61, 61)], 6, 2, 64, 4)


@pytest.mark.parametrize("key_groups", [1, 2])
@pytest.mark.parametrize("window", [1, 7, 64, 100])
def test_attention_prefill_window(window, key_groups):
    got, want = _prefill([(260, 260), (300, 40)], 4, 2, 64, 8, window=window, key_groups=key_groups)
    torch.testing.assert_close(got, want, rtol=2 ** -6, atol=2 ** -6)


def test_attention_prefill_sharp_scores_find_the_right_key():
    """Each query matches exactly one key (its own position minus a fixed distance): a kernel that
    mixes up tiles, pages or the causal edge returns another key's value."""
    hq, hkv, dh, page, S = 8, 2, 128, 16, 400
    torch.manual_seed(0)
    dirs = torch.randn(S, dh)
    dirs /= dirs.norm(dim=-1, keepdim=True)
    v = torch.randn(S, hkv, dh).bfloat16()
    ops = _ops()
    for dist in (0, 1, 63, 64, 200):
        k = (dirs * 12)[:, None, :].expand(S, hkv, dh).bfloat16()
        tgt = (torch.arange(S) - dist).clamp(min=0)
        q = (dirs[tgt] * 12 * math.sqrt(dh) / 4)[:, None, :].expand(S, hq, dh).bfloat16()
        n_pages = -(-S // page) + 2
        k_pages, v_pages, table = _paged(k, v, page, n_pages, dtype=torch.bfloat16)
        qpt = ops.prefill_queries_per_tile(hq, hkv, dh)
        trow, tq0 = ops.prefill_tiles([0, S], 0, 1, qpt)
        want = v[tgt].float().repeat_interleave(hq // hkv, dim=1).reshape(S, hq * dh)
        for key_groups in (1, 2):
            out = torch.zeros(S, hq * dh, dtype=torch.bfloat16, device=DEV)
            ops.attention_prefill(q.reshape(S, hq * dh).to(DEV), hq, hkv, dh, k_pages, v_pages, _i32([0, S]), _i32([S]), _i32([table]),
                                  _i32(trow), _i32(tq0), 0, dh ** -0.5, out, key_groups=key_groups)
            err = (out.float().cpu() - want).abs().amax(dim=1)
            assert err.max().item() < 3e-2, f"distance {dist}, {key_groups} key groups: first bad query {int((err >= 3e-2).nonzero()[0])}"


@pytest.mark.parametrize("key_groups", [1, 2])
def test_attention_prefill_behind_a_prefix_of_32768_keys(key_groups):
    """Two tile rows of new tokens behind 32,704 cached ones: 512 tiles of keys a block, block tables
    of 2,048 pages.  Random scores first; then every query matches exactly one key, at a fixed
    distance that reaches from its own position to the first pages of the prefix."""
    ops = _ops()
    hq, hkv, dh, page, S, sq = 32, 8, 128, 16, 32768, 64
    g = torch.Generator().manual_seed(5)
    n_pages = S // page + 4
    table = torch.randperm(n_pages, generator=g)[: S // page].tolist()
    qpt = ops.prefill_queries_per_tile(hq, hkv, dh)
    trow, tq0 = ops.prefill_tiles([0, sq], 0, 1, qpt, [S])
    assert len(trow) == 2

    def run(q, k, v):
        k_pages = torch.full((n_pages, hkv, page, dh), 40.0, dtype=torch.bfloat16)
        v_pages = torch.full((n_pages, hkv, page, dh), -40.0, dtype=torch.bfloat16)
        _fill_pages(k_pages, v_pages, table, k, v)
        out = torch.zeros(sq, hq * dh, dtype=torch.bfloat16, device=DEV)
        ops.attention_prefill(q.reshape(sq, hq * dh).to(DEV), hq, hkv, dh, k_pages.to(DEV), v_pages.to(DEV), _i32([0, sq]), _i32([S]),
                              _i32([table]), _i32(trow), _i32(tq0), 0, dh ** -0.5, out, key_groups=key_groups)
        return out.float().cpu()

    k = (torch.randn(S, hkv, dh, generator=g) * 0.5).bfloat16()
    v = torch.randn(S, hkv, dh, generator=g).bfloat16()
    q = (torch.randn(sq, hq, dh, generator=g) * 2).bfloat16()
    want = plain.attention(q.float().to(DEV), k.float().to(DEV), v.float().to(DEV)).cpu()
    torch.testing.assert_close(run(q, k, v), want, rtol=2 ** -6, atol=2 ** -6)

    dirs = torch.randn(S, dh, generator=g)
    dirs /= dirs.norm(dim=-1, keepdim=True)
    k = (dirs * 12)[:, None, :].expand(S, hkv, dh).bfloat16()
    for dist in (0, 1, 63, 64, 8191, 20000, S - sq):
        tgt = torch.arange(S - sq, S) - dist
        q = (dirs[tgt] * 12 * math.sqrt(dh) / 3)[:, None, :].expand(sq, hq, dh).bfloat16()
        got = run(q, k, v)
        err = (got - v[tgt].float().repeat_interleave(hq // hkv, dim=1).reshape(sq, hq * dh)).abs().amax(dim=1)
        assert err.max().item() < 3e-2, f"distance {dist}: first bad query {int((err >= 3e-2).nonzero()[0])}"
