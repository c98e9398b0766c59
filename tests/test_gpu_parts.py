"""Each part alone on the GPU against its plain counterpart, and a toy mixer with state of its own
that is registered, built and stepped without a change to the framework's files."""


import pytest
import torch
import torch.nn.functional as F

from .helpers import random_tokens
from .plain import llama as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _ctx_and_cache(n_tokens, hkv, dh, page, dtype, start=0):
    """A one-request step context and cache for ``n_tokens`` new tokens after ``start`` cached ones."""
    from torchllms_amd.cache import CacheGroupSpec, CacheManager
    from torchllms_amd.engine.context import upload
    from torchllms_amd.engine.layout import StepEntry, build_step_layout

    cache = CacheManager([CacheGroupSpec("kv0", (0,), hkv, dh)], [], page, 64, 2, dtype=dtype, device=DEV)
    cache.admit("r")
    return cache


def _step(cache, rid, n_tokens, want=()):
    from torchllms_amd.engine.context import upload
    from torchllms_amd.engine.layout import StepEntry, build_step_layout

    e = StepEntry(rid, [0] * n_tokens, list(want))
    start = cache.extend(rid, n_tokens)
    lay = build_step_layout([e], [start], [cache.slot(rid)], [[cache.block_table(rid, g)] for g in range(len(cache.groups))], cache.page_size)
    return upload(lay, DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_part_whole_and_in_portions(dtype):
    from torchllms_amd.config.spec import PartSpec
    from torchllms_amd.kernels import ops
    from torchllms_amd.parts import MIXERS

    torch.manual_seed(0)
    D, hq, hkv, dh, S = 80, 5, 1, 24, 29
    scaling = {"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0, "high_freq_factor": 2.0, "original_max_position_embeddings": 16}
    spec = PartSpec("attention", dict(hidden_size=D, num_heads=hq, num_kv_heads=hkv, head_dim=dh, qkv_bias=True,
                                      softmax_scale=dh ** -0.5, window=0,
                                      position=PartSpec("rope", dict(head_dim=dh, rotary_dim=dh, theta=777.0, scaling=scaling))))
    part = MIXERS.build(spec)
    assert part.cache_need().num_kv_heads == 1 and part.cache_need().head_dim == 24
    w = {n: (torch.randn(s.shape) * (0.3 if len(s.shape) == 2 else 0.1)).to(dtype) for n, s in part.param_specs().items()}
    assert set(w) == {"wq.weight", "wk.weight", "wv.weight", "wo.weight", "wq.bias", "wk.bias", "wv.bias"}
    part.bind({k: v.to(DEV) for k, v in w.items()})
    x = torch.randn(S, D).to(dtype)
    # plain: interleaved rotation on the weights as given (the part's own layout)
    f = plain.rope_inverse_frequencies(dh, 777.0, scaling)
    pos = torch.arange(S)

    def plain_part(dt):
        xx, ww = x.to(dt), {k: v.to(dt) for k, v in w.items()}
        q = plain.rope_rotate_interleaved(F.linear(xx, ww["wq.weight"], ww["wq.bias"]).view(S, hq, dh), pos, f)
        k = plain.rope_rotate_interleaved(F.linear(xx, ww["wk.weight"], ww["wk.bias"]).view(S, hkv, dh), pos, f)
        v = F.linear(xx, ww["wv.weight"], ww["wv.bias"]).view(S, hkv, dh)
        return F.linear(plain.attention(q, k, v), ww["wo.weight"]).float(), k.float()

    want, k = plain_part(torch.float32)
    if dtype == torch.float32:
        tol = dict(rtol=1e-4, atol=1e-4)
    else:  # the yardstick is the plain part computed in bfloat16
        tol = dict(rtol=0.0, atol=2 * (plain_part(torch.bfloat16)[0] - want).abs().max().item())
    for cuts in ([S], [11, 2, 1, 15]):
        cache = _ctx_and_cache(S, hkv, dh, 8, dtype)
        outs, at = [], 0
        for n in cuts:
            ctx = _step(cache, "r", n)
            # (a mixer may leave its last product to whoever adds it to the residual stream)
            outs.append(ops.resolved(part.forward(x[at : at + n].to(DEV).contiguous(), ctx, cache.kv_view(0))))
            cache.advance("r", n)
            at += n
        torch.testing.assert_close(torch.cat(outs).float().cpu(), want, **tol)
        kk, vv = cache.gather_kv("r", 0)
        torch.testing.assert_close(kk.float().cpu(), k, **(tol if dtype == torch.float32 else dict(rtol=0.02, atol=0.05)))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_norm_embedding_head_and_block(dtype):
    from torchllms_amd.config.spec import PartSpec
    from torchllms_amd.kernels import ops
    from torchllms_amd.parts import BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS

    torch.manual_seed(1)
    D, Fi, V, S = 72, 200, 131, 13
    tol = dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32 else dict(rtol=0.05, atol=0.1)
    ffn = FEED_FORWARDS.build(PartSpec("swiglu", dict(hidden_size=D, intermediate_size=Fi)))
    w = {n: (torch.randn(s.shape) * 0.2).to(dtype) for n, s in ffn.param_specs().items()}
    ffn.bind({k: v.to(DEV) for k, v in w.items()})
    x = torch.randn(S, D).to(dtype)
    want = plain.swiglu(x.float(), w["w1.weight"].float(), w["w3.weight"].float(), w["w2.weight"].float())
    torch.testing.assert_close(ops.resolved(ffn.forward(x.to(DEV), None)).float().cpu(), want, **tol)

    norm = NORMS.build(PartSpec("rmsnorm", dict(size=D, eps=1e-3)))
    nw = (1 + 0.2 * torch.randn(D)).to(dtype)
    norm.bind({"weight": nw.to(DEV)})
    torch.testing.assert_close(norm.forward(x.to(DEV)).float().cpu(), plain.rms_norm(x, nw, 1e-3).float(), **tol)
    d = torch.randn(S, D).to(dtype)
    h2, y2 = norm.forward_add(x.to(DEV), d.to(DEV))
    assert torch.equal(h2.cpu(), x + d)
    torch.testing.assert_close(y2.float().cpu(), plain.rms_norm(x + d, nw, 1e-3).float(), **tol)

    emb = EMBEDDINGS.build(PartSpec("embedding", dict(vocab_size=V, hidden_size=D)))
    table = torch.randn(V, D).to(dtype)
    emb.bind({"weight": table.to(DEV)})
    toks = torch.tensor(random_tokens(S, V, 0), dtype=torch.int32)
    assert torch.equal(emb.forward(toks.to(DEV)).cpu(), table[toks.long()])
    for tied in (True, False):
        head = HEADS.build(PartSpec("lm_head", dict(vocab_size=V, hidden_size=D, tied=tied)))
        hw = torch.randn(V, D).to(dtype) * 0.2
        if tied:
            assert head.param_specs() == {}
            head.tie(emb)
            hw = table
        else:
            head.bind({"weight": hw.to(DEV)})
        logits = head.forward(x.to(DEV))
        assert logits.dtype == torch.float32
        torch.testing.assert_close(logits.cpu(), F.linear(x.float(), hw.float()), **(tol if dtype == torch.float32 else dict(rtol=0.05, atol=0.5)))


def test_pre_norm_block_matches_the_plain_block():
    from torchllms_amd.config.spec import PartSpec
    from torchllms_amd.parts import BLOCKS, FEED_FORWARDS, MIXERS, NORMS

    torch.manual_seed(2)
    cfg = dict(hidden_size=48, num_attention_heads=3, num_key_value_heads=3, head_dim=16, intermediate_size=100, rms_norm_eps=1e-5)
    D, S = 48, 17
    pos_spec = PartSpec("rope", dict(head_dim=16, rotary_dim=16, theta=10000.0, scaling=None))
    block = BLOCKS["pre_norm"](
        {
            "mixer": MIXERS.build(PartSpec("attention", dict(hidden_size=D, num_heads=3, num_kv_heads=3, head_dim=16, qkv_bias=False,
                                                             softmax_scale=0.25, window=0, position=pos_spec))),
            "ffn": FEED_FORWARDS.build(PartSpec("swiglu", dict(hidden_size=D, intermediate_size=100))),
            "mixer_norm": NORMS.build(PartSpec("rmsnorm", dict(size=D, eps=1e-5))),
            "ffn_norm": NORMS.build(PartSpec("rmsnorm", dict(size=D, eps=1e-5))),
        }
    )
    w = {n: (torch.randn(s.shape) * 0.3 if s.init == "normal" else 1 + 0.1 * torch.randn(s.shape)) for n, s in block.param_specs().items()}
    block.bind({k: v.to(DEV) for k, v in w.items()})
    lw = {"wq": w["mixer.wq.weight"], "wk": w["mixer.wk.weight"], "wv": w["mixer.wv.weight"], "wo": w["mixer.wo.weight"],
          "w1": w["ffn.w1.weight"], "w3": w["ffn.w3.weight"], "w2": w["ffn.w2.weight"],
          "attention_norm": w["mixer_norm.weight"], "ffn_norm": w["ffn_norm.weight"]}
    x = torch.randn(S, D)
    want = plain.block(x, lw, cfg, torch.arange(S), plain.rope_inverse_frequencies(16, 10000.0, None))
    cache = _ctx_and_cache(S, 3, 16, 4, torch.float32)
    ctx = _step(cache, "r", S)
    h, delta = block.forward(x.to(DEV), None, ctx, {"mixer": cache.kv_view(0)})
    torch.testing.assert_close((h + delta).cpu(), want, rtol=1e-4, atol=1e-4)
    # a pending delta from the layer before is added first
    cache2 = _ctx_and_cache(S, 3, 16, 4, torch.float32)
    h2, d2 = block.forward((x * 0.5).to(DEV), (x * 0.5).to(DEV), _step(cache2, "r", S), {"mixer": cache2.kv_view(0)})
    torch.testing.assert_close((h2 + d2).cpu(), want, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("intermediate", [104, 100])
def test_pre_norm_blocks_in_bfloat16_leave_their_norms_to_the_products(intermediate):
    """On bfloat16 steps of few rows the products do the norms' work: the product that ends a branch
    adds it to the residual stream and leaves the rows' statistics, the product that reads the rows
    (times the norm's gain) applies them.  Two blocks
    in a row against the plain blocks, with few rows (fused) and with many (the norm kernel), which
    agree with each other too.  An intermediate size that the weight-streaming kernel does not take
    (100, no multiple of 8) leaves that product, and the norm behind it, to the other kernels."""
    from torchllms_amd.config.spec import PartSpec
    from torchllms_amd.kernels import ops
    from torchllms_amd.parts import BLOCKS, FEED_FORWARDS, MIXERS, NORMS

    torch.manual_seed(7)
    D, hq, hkv, dh, eps = 80, 5, 1, 16, 1e-2
    cfg = dict(hidden_size=D, num_attention_heads=hq, num_key_value_heads=hkv, head_dim=dh, intermediate_size=intermediate, rms_norm_eps=eps)
    pos_spec = PartSpec("rope", dict(head_dim=dh, rotary_dim=dh, theta=10000.0, scaling=None))
    blocks, weights = [], []
    for _ in range(2):
        block = BLOCKS["pre_norm"](
            {
                "mixer": MIXERS.build(PartSpec("attention", dict(hidden_size=D, num_heads=hq, num_kv_heads=hkv, head_dim=dh, qkv_bias=False,
                                                                 softmax_scale=dh ** -0.5, window=0, position=pos_spec))),
                "ffn": FEED_FORWARDS.build(PartSpec("swiglu", dict(hidden_size=D, intermediate_size=intermediate))),
                "mixer_norm": NORMS.build(PartSpec("rmsnorm", dict(size=D, eps=eps))),
                "ffn_norm": NORMS.build(PartSpec("rmsnorm", dict(size=D, eps=eps))),
            }
        )
        # gains far from one, so that a gain applied twice or not at all shows
        w = {n: ((torch.randn(s.shape) * 0.15) if s.init == "normal" else (0.3 + torch.rand(s.shape) * 2.0)).bfloat16() for n, s in block.param_specs().items()}
        block.bind({k: v.to(DEV) for k, v in w.items()})
        blocks.append(block)
        weights.append({"wq": w["mixer.wq.weight"], "wk": w["mixer.wk.weight"], "wv": w["mixer.wv.weight"], "wo": w["mixer.wo.weight"],
                        "w1": w["ffn.w1.weight"], "w3": w["ffn.w3.weight"], "w2": w["ffn.w2.weight"],
                        "attention_norm": w["mixer_norm.weight"], "ffn_norm": w["ffn_norm.weight"]})
    seen = []
    for block in blocks:
        for part in (block.mixer, block.ffn):
            def spy(x, *rest, _inner=part.forward):
                seen.append(type(x).__name__)
                return _inner(x, *rest)
            part.forward = spy

    def run(S):
        x = (torch.randn(S, D, generator=torch.Generator().manual_seed(S)) * 2).bfloat16()
        want = x.float()
        for lw in weights:
            want = plain.block(want, {k: v.float() for k, v in lw.items()}, cfg, torch.arange(S), plain.rope_inverse_frequencies(dh, 10000.0, None))
        h, delta = x.to(DEV), None
        del seen[:]
        for i, block in enumerate(blocks):
            cache = _ctx_and_cache(S, hkv, dh, 4, torch.bfloat16)
            h, delta = block.forward(h, delta, _step(cache, "r", S), {"mixer": cache.kv_view(0)})
        got = h.float() + ops.resolved(delta).float()
        torch.testing.assert_close(got.cpu(), want, rtol=0.05, atol=0.03 * want.abs().max().item())
        return x, got.cpu(), list(seen)

    x, few, kinds = run(7)
    streamed = intermediate % 8 == 0  # whether the product back to the model's width takes the weight-streaming kernel
    assert kinds == ["Tensor", "NormedRows", "NormedRows" if streamed else "Tensor", "NormedRows"]
    _, many, kinds = run(40)
    assert kinds == ["Tensor"] * 4
