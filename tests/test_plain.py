"""Pins the plain implementation (tests/plain/llama.py) by what fixes it beside the reference's
text: special cases that reduce to a library routine, invariants, and the vectors the reference's
own tests hold.  Each check is chosen so that a plausible mistake fails it.  CPU only."""

import math

import pytest
import torch
import torch.nn.functional as F

from .helpers import TINY_A, TINY_B, TINY_C, random_tokens
from .plain import llama as plain


# ----------------------------------------------------------------------------- RMS norm
def test_rms_norm_formula():
    torch.manual_seed(0)
    x = torch.randn(5, 48)
    w = torch.randn(48)
    want = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5) * w
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), want, atol=1e-6)


def test_rms_norm_constant_row_and_eps_placement():
    # a constant row c gives c / sqrt(c^2 + eps): eps inside the root, added to the mean
    for c, eps in [(1e-3, 1e-5), (1e-3, 1e-6), (2.0, 1e-5)]:
        x = torch.full((1, 32), c)
        got = plain.rms_norm(x, torch.ones(32), eps)[0, 0].item()
        assert got == pytest.approx(c / math.sqrt(c * c + eps), rel=1e-5)
    # the two eps of the tiny configurations are told apart on a small row
    x = torch.full((1, 32), 1e-3)
    a = plain.rms_norm(x, torch.ones(32), 1e-5)[0, 0].item()
    b = plain.rms_norm(x, torch.ones(32), 1e-6)[0, 0].item()
    assert abs(a - b) > 0.1
    assert torch.equal(plain.rms_norm(torch.zeros(1, 8), torch.ones(8), 1e-5), torch.zeros(1, 8))


def test_rms_norm_casts_before_the_weight():
    # in bfloat16 the normalised value is rounded first, then multiplied: bf16(bf16(n) * w)
    torch.manual_seed(1)
    x = torch.randn(3, 64).bfloat16()
    w = (1 + 0.3 * torch.randn(64)).bfloat16()
    xf = x.float()
    n = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)).bfloat16()
    assert torch.equal(plain.rms_norm(x, w, 1e-5), n * w)
    fused = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5) * w.float()).bfloat16()
    assert not torch.equal(fused, n * w)  # the other order of rounding is a different function


# ----------------------------------------------------------------------------- rotary
def test_rope_default_frequencies():
    f = plain.rope_inverse_frequencies(16, 10000.0, None)
    want = torch.tensor([10000.0 ** (-2 * i / 16) for i in range(8)])
    assert torch.allclose(f, want, rtol=1e-6)
    assert f[0] == 1.0


def test_rope_position_zero_is_identity_and_norms_are_kept():
    torch.manual_seed(0)
    x = torch.randn(6, 3, 16)
    f = plain.rope_inverse_frequencies(16, 10000.0, None)
    pos = torch.arange(6)
    y = plain.rope_rotate_interleaved(x, pos, f)
    assert torch.equal(y[0], x[0])
    pair_norm = lambda t: t.reshape(6, 3, 8, 2).pow(2).sum(-1)
    assert torch.allclose(pair_norm(y), pair_norm(x), atol=1e-5)


def test_rope_direction_and_pairing():
    # pair (1, 0) at position 1 with frequency f turns into (cos f, sin f): counter-clockwise,
    # and it is the neighbours (2i, 2i+1) that form a pair
    f = torch.tensor([0.5, 0.25])
    x = torch.tensor([[[1.0, 0.0, 0.0, 1.0]]])
    y = plain.rope_rotate_interleaved(x, torch.tensor([1]), f)[0, 0]
    want = torch.tensor([math.cos(0.5), math.sin(0.5), -math.sin(0.25), math.cos(0.25)])
    assert torch.allclose(y, want, atol=1e-6)
    # the same as multiplying complex numbers
    torch.manual_seed(3)
    x = torch.randn(5, 2, 8)
    f = plain.rope_inverse_frequencies(8, 100.0, None)
    pos = torch.tensor([0, 3, 4, 9, 17])
    z = torch.view_as_complex(x.reshape(5, 2, 4, 2)) * torch.polar(torch.ones(5, 4), torch.outer(pos.float(), f))[:, None]
    assert torch.allclose(plain.rope_rotate_interleaved(x, pos, f), torch.view_as_real(z).reshape(5, 2, 8), atol=1e-5)


def test_rope_scores_depend_on_distance_only():
    torch.manual_seed(0)
    q = torch.randn(1, 1, 32)
    k = torch.randn(1, 1, 32)
    f = plain.rope_inverse_frequencies(32, 500000.0, TINY_B["rope_scaling"])

    def score(m, n):
        a = plain.rope_rotate_interleaved(q, torch.tensor([m]), f)
        b = plain.rope_rotate_interleaved(k, torch.tensor([n]), f)
        return (a * b).sum().item()

    assert score(7, 3) == pytest.approx(score(47, 43), abs=1e-4)
    assert score(7, 3) != pytest.approx(score(7, 4), abs=1e-4)


def test_rope_llama3_bands():
    sc = TINY_B["rope_scaling"]  # factor 8, low 1, high 4, original 64
    base = plain.rope_inverse_frequencies(32, 500000.0, None)
    got = plain.rope_inverse_frequencies(32, 500000.0, sc)
    wl = 2 * math.pi / base
    short = wl < 64 / 4
    long = wl > 64 / 1
    assert short.any() and long.any() and (~short & ~long).any()
    assert torch.equal(got[short], base[short])  # short wavelengths untouched
    assert torch.allclose(got[long], base[long] / 8, rtol=1e-6)  # long ones divided by the factor
    mid = ~short & ~long
    assert ((got[mid] < base[mid]) & (got[mid] > base[mid] / 8)).all()
    assert (got[1:] <= got[:-1]).all()  # still non-increasing
    one = dict(sc, factor=1.0)
    assert torch.allclose(plain.rope_inverse_frequencies(32, 500000.0, one), base, rtol=1e-6)
    with pytest.raises(ValueError, match="Unknown RoPE type"):
        plain.rope_inverse_frequencies(32, 1e4, {"rope_type": "yarn"})


def _both_frequency_functions():
    from torchllms_amd.parts.positions import rotary_inverse_frequencies

    return [("plain", plain.rope_inverse_frequencies), ("engine", rotary_inverse_frequencies)]


@pytest.mark.parametrize("factor, low, high, old", [(8.0, 1.0, 4.0, 8192), (32.0, 1.0, 4.0, 8192), (4.0, 2.0, 3.0, 640)])
def test_rope_llama3_blend_is_continuous_linear_and_ends_where_the_bands_say(factor, low, high, old):
    """What fixes the middle band beside the reference's text: on a dense grid of frequencies
    (2,048 of them, from sixty to hundreds inside the band) the ratio scaled / unscaled is 1 for wavelengths below
    old/high, 1/factor above old/low, and in between it moves from the one to the other without a
    jump, rising with x = old / wavelength, with one slope everywhere (linear in x).  Swapped blend
    weights, or low and high exchanged, put the values of the two outer bands at the wrong edges:
    a jump of (1 - 1/factor) at each (reference: networks.py:259-277).  Both the plain function and
    the engine's own are asked."""
    sc = {"rope_type": "llama3", "factor": factor, "low_freq_factor": low, "high_freq_factor": high,
          "original_max_position_embeddings": old}
    dim, theta = 4096, 500000.0
    for name, fn in _both_frequency_functions():
        base = fn(dim, theta, None).double()
        got = fn(dim, theta, sc).double()
        x = old * base / (2 * math.pi)  # old / wavelength, falling along the grid
        ratio = got / base
        short, long = x > high, x < low
        band = ~short & ~long
        assert band.sum() > 50 and short.sum() > 100 and long.sum() > 100, name
        assert torch.allclose(ratio[short], torch.ones_like(ratio[short]), rtol=1e-6), name
        assert torch.allclose(ratio[long], torch.full_like(ratio[long], 1 / factor), rtol=1e-6), name
        # no jump anywhere: neighbours on the grid differ by at most what the slope allows
        slope = (1 - 1 / factor) / (high - low)
        steps = (x[:-1] - x[1:]).abs()
        jumps = (ratio[:-1] - ratio[1:]).abs()
        assert (jumps <= slope * steps * 1.01 + 1e-6).all(), f"{name}: a jump of {jumps.max().item()} at x = {x[jumps.argmax()].item()}"
        # rising with x inside the band, with the same slope between any two neighbours
        xb, rb = x[band], ratio[band]
        local = (rb[:-1] - rb[1:]) / (xb[:-1] - xb[1:])
        assert torch.allclose(local, torch.full_like(local, slope), rtol=2e-3), f"{name}: slopes {local.min().item()}..{local.max().item()}, expected {slope}"
        # and anchored: the value at the band's middle is the mean of the two outer values
        mid = (xb - (low + high) / 2).abs().argmin()
        assert rb[mid].item() == pytest.approx((1 + 1 / factor) / 2 + slope * (xb[mid].item() - (low + high) / 2), rel=1e-5), name


def test_rope_llama3_middle_band_numbers_worked_out_by_hand():
    """Llama 3.1's own constants (theta 500000, head size 128, factor 8, low 1, high 4, old 8192), pair
    i has theta_i = 500000^(-2i/128) and wavelength 2 pi / theta_i.  From the reference's lines
    (networks.py:259-277), with a pocket calculator:
      i = 28: wavelength 1956.5 < 2048               -> untouched
      i = 29: wavelength 2401.7, smooth = (8192/2401.7 - 1)/3 = 0.80362 -> ratio (1-s)/8 + s = 0.828168
      i = 31: wavelength 3619.2, smooth = 0.42115                        -> ratio 0.493507
      i = 34: wavelength 6695.1, smooth = 0.074527                       -> ratio 0.190211
      i = 35: wavelength 8218.7 > 8192               -> divided by 8
    """
    sc = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
          "original_max_position_embeddings": 8192}
    want = {28: 0.003211446, 29: 0.0026160993 * 0.828168412, 31: 0.0017360467 * 0.493507123, 34: 0.00093847387 * 0.190210744,
            35: 0.00076449699 / 8}
    assert want[29] == pytest.approx(0.00216657076, rel=1e-7) and want[34] == pytest.approx(0.000178507813, rel=1e-7)
    for name, fn in _both_frequency_functions():
        got = fn(128, 500000.0, sc)
        assert got.dtype == torch.float32
        for i, value in want.items():
            assert got[i].item() == pytest.approx(value, rel=2e-6), f"{name}: pair {i}"


def test_row_permutation_matches_the_other_pairing():
    # half-split rotation of unpermuted vectors and interleaved rotation of permuted ones give the
    # same scores (reference: checkpoint_converter.py:96-108)
    torch.manual_seed(0)
    H, dh, S = 3, 8, 5
    q = torch.randn(S, H * dh)
    k = torch.randn(S, H * dh)
    f = plain.rope_inverse_frequencies(dh, 10000.0, None)
    pos = torch.arange(S) + 2
    perm = lambda t: plain.permute_rows_for_interleaved(t.T.contiguous(), H, dh).T
    a = plain.rope_rotate_half_split(q.view(S, H, dh), pos, f)
    b = plain.rope_rotate_half_split(k.view(S, H, dh), pos, f)
    c = plain.rope_rotate_interleaved(perm(q).reshape(S, H, dh), pos, f)
    d = plain.rope_rotate_interleaved(perm(k).reshape(S, H, dh), pos, f)
    assert torch.allclose(torch.einsum("shd,thd->hst", a, b), torch.einsum("shd,thd->hst", c, d), atol=1e-5)
    # explicit small case: head of size 4, rows [a0 a1 | b0 b1] -> [a0 b0 a1 b1]
    w = torch.arange(8.0).reshape(8, 1)
    assert plain.permute_rows_for_interleaved(w, 2, 4).flatten().tolist() == [0, 2, 1, 3, 4, 6, 5, 7]


# ----------------------------------------------------------------------------- attention
@pytest.mark.parametrize("hq, hkv", [(4, 4), (4, 2), (6, 1)])
def test_attention_whole_prompt_is_sdpa(hq, hkv):
    torch.manual_seed(0)
    S, dh = 9, 8
    q, k, v = torch.randn(S, hq, dh), torch.randn(S, hkv, dh), torch.randn(S, hkv, dh)
    want = F.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None], is_causal=True, enable_gqa=hq != hkv
    )[0].transpose(0, 1).reshape(S, hq * dh)
    assert torch.allclose(plain.attention(q, k, v), want, atol=1e-5)


def test_attention_with_prefix_matches_the_references_own_vector():
    # reference: torchllms/inference/test_prefix_cache_wiring.py:238-254: bsz 2, qlen 3, past 2,
    # 2 heads, head size 4, seed 0, shifted causal mask, max diff < 1e-5
    torch.manual_seed(0)
    bsz, qlen, past, h, d = 2, 3, 2, 2, 4
    xq = torch.randn(bsz, qlen, h, d)
    xk = torch.randn(bsz, qlen + past, h, d)
    xv = torch.randn(bsz, qlen + past, h, d)
    mask = torch.zeros(qlen, qlen + past, dtype=torch.bool)
    for i in range(qlen):
        mask[i, : past + i + 1] = True
    for b in range(bsz):
        want = F.scaled_dot_product_attention(
            xq[b].transpose(0, 1)[None], xk[b].transpose(0, 1)[None], xv[b].transpose(0, 1)[None], attn_mask=mask
        )[0].transpose(0, 1).reshape(qlen, h * d)
        assert (plain.attention(xq[b], xk[b], xv[b]) - want).abs().max() < 1e-5


def test_attention_limits():
    torch.manual_seed(0)
    q, k, v = torch.randn(1, 4, 8), torch.randn(1, 2, 8), torch.randn(1, 2, 8)
    # one token: the output is v of the head's group
    out = plain.attention(q, k, v).view(4, 8)
    assert torch.allclose(out, v[0].repeat_interleave(2, dim=0), atol=1e-6)
    # all values equal within a group: the output is that value; query head h reads group h // 2
    S = 7
    q = torch.randn(S, 4, 8)
    k = torch.randn(S, 2, 8)
    v = torch.stack([torch.full((S, 8), 3.0), torch.full((S, 8), -5.0)], dim=1)
    out = plain.attention(q, k, v).view(S, 4, 8)
    assert torch.allclose(out[:, 0], torch.full((S, 8), 3.0)) and torch.allclose(out[:, 1], torch.full((S, 8), 3.0))
    assert torch.allclose(out[:, 2], torch.full((S, 8), -5.0)) and torch.allclose(out[:, 3], torch.full((S, 8), -5.0))


def test_attention_is_causal_and_scaled():
    torch.manual_seed(0)
    S, dh = 6, 16
    q, k, v = torch.randn(S, 1, dh), torch.randn(S, 1, dh), torch.randn(S, 1, dh)
    base = plain.attention(q, k, v)
    k2, v2 = k.clone(), v.clone()
    k2[4:], v2[4:] = 9.0, 9.0  # the future must not reach queries 0..3
    assert torch.equal(plain.attention(q, k2, v2)[:4], base[:4])
    # scale is 1/sqrt(dh): a far key made to stand out by that scale dominates
    w = torch.softmax((q[-1, 0] @ k[:, 0].T) / math.sqrt(dh), -1)
    assert torch.allclose(base[-1], w @ v[:, 0], atol=1e-5)
    assert torch.allclose(plain.attention(q, k, v, scale=dh ** -0.5), base, atol=1e-6)


# ----------------------------------------------------------------------------- feed-forward
def test_swiglu():
    torch.manual_seed(0)
    x, w1, w3, w2 = torch.randn(4, 12), torch.randn(20, 12), torch.randn(20, 12), torch.randn(12, 20)
    g = x @ w1.T
    want = ((g * torch.sigmoid(g)) * (x @ w3.T)) @ w2.T
    assert torch.allclose(plain.swiglu(x, w1, w3, w2), want, atol=1e-5)
    # gate and up are not interchangeable
    assert not torch.allclose(plain.swiglu(x, w3, w1, w2), want, atol=1e-3)


# ----------------------------------------------------------------------------- whole model
def _weights(cfg, seed=0):
    torch.manual_seed(seed)
    hq = cfg["num_attention_heads"]
    hkv = cfg.get("num_key_value_heads") or hq
    dh = cfg.get("head_dim") or cfg["hidden_size"] // hq
    D, Fi, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    w = {"model.embed_tokens.weight": torch.randn(V, D) * 0.5, "model.norm.weight": 1 + 0.1 * torch.randn(D)}
    if not cfg.get("tie_word_embeddings"):
        w["lm_head.weight"] = torch.randn(V, D) * 0.1
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        w[p + "self_attn.q_proj.weight"] = torch.randn(hq * dh, D) * 0.2
        w[p + "self_attn.k_proj.weight"] = torch.randn(hkv * dh, D) * 0.2
        w[p + "self_attn.v_proj.weight"] = torch.randn(hkv * dh, D) * 0.2
        w[p + "self_attn.o_proj.weight"] = torch.randn(D, hq * dh) * 0.2
        w[p + "mlp.gate_proj.weight"] = torch.randn(Fi, D) * 0.2
        w[p + "mlp.up_proj.weight"] = torch.randn(Fi, D) * 0.2
        w[p + "mlp.down_proj.weight"] = torch.randn(D, Fi) * 0.2
        w[p + "input_layernorm.weight"] = 1 + 0.1 * torch.randn(D)
        w[p + "post_attention_layernorm.weight"] = 1 + 0.1 * torch.randn(D)
        if cfg.get("attention_bias"):
            w[p + "self_attn.q_proj.bias"] = torch.randn(hq * dh) * 0.1
            w[p + "self_attn.k_proj.bias"] = torch.randn(hkv * dh) * 0.1
            w[p + "self_attn.v_proj.bias"] = torch.randn(hkv * dh) * 0.1
    return w


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B, TINY_C], ids=["A", "B", "C"])
def test_forward_depends_on_distances_only(cfg):
    w = _weights(cfg)
    toks = random_tokens(12, cfg["vocab_size"], 1)
    a = plain.forward(w, cfg, toks)
    b = plain.forward(w, cfg, toks, start_position=37)
    assert a.shape == (12, cfg["vocab_size"])
    assert torch.allclose(a, b, atol=2e-4)


def test_forward_is_causal_and_prefix_stable():
    w = _weights(TINY_A)
    toks = random_tokens(10, 256, 2)
    full = plain.forward(w, TINY_A, toks)
    part = plain.forward(w, TINY_A, toks[:6])
    assert torch.allclose(full[:6], part, atol=1e-5)


def test_forward_tied_output_is_the_embedding_matrix():
    w = _weights(TINY_A)
    assert "lm_head.weight" not in w
    toks = random_tokens(4, 256, 3)
    logits = plain.forward(w, TINY_A, toks)
    # the same model spelled untied, with the output matrix a copy of the embedding matrix
    untied = dict(TINY_A, tie_word_embeddings=False)
    w2 = dict(w)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    assert torch.equal(plain.forward(w2, untied, toks), logits)
    # and an output matrix that is present is ignored when the configuration ties
    w2["lm_head.weight"] = torch.zeros_like(w2["lm_head.weight"])
    assert torch.equal(plain.forward(w2, TINY_A, toks), logits)


def test_forward_one_layer_by_hand():
    cfg = dict(TINY_C)
    w = _weights(cfg)
    toks = random_tokens(5, cfg["vocab_size"], 4)
    lw = plain.layer_weights(w, 0, cfg)
    x = w["model.embed_tokens.weight"][torch.tensor(toks)]
    pos = torch.arange(5)
    f = plain.rope_inverse_frequencies(48, cfg["rope_theta"], cfg["rope_scaling"])
    n1 = plain.rms_norm(x, lw["attention_norm"], cfg["rms_norm_eps"])
    q = (n1 @ lw["wq"].T + lw["bq"]).view(5, 6, 48)
    k = (n1 @ lw["wk"].T + lw["bk"]).view(5, 3, 48)
    v = (n1 @ lw["wv"].T + lw["bv"]).view(5, 3, 48)
    q, k = plain.rope_rotate_interleaved(q, pos, f), plain.rope_rotate_interleaved(k, pos, f)
    h = x + plain.attention(q, k, v) @ lw["wo"].T
    out = h + plain.swiglu(plain.rms_norm(h, lw["ffn_norm"], cfg["rms_norm_eps"]), lw["w1"], lw["w3"], lw["w2"])
    logits = plain.rms_norm(out, w["model.norm.weight"], cfg["rms_norm_eps"]) @ w["lm_head.weight"].T
    assert torch.allclose(plain.forward(w, cfg, toks), logits, atol=1e-5)


# ----------------------------------------------------------------------------- sampling
def test_sampling_rules():
    torch.manual_seed(0)
    logits = torch.randn(3, 50)
    q = torch.empty(3, 50).exponential_(1)
    assert torch.equal(plain.sample_with_exponentials(logits, 0.0, q), logits.argmax(-1))
    assert torch.equal(plain.sample_with_exponentials(logits, 1e-7, q), logits.argmax(-1))
    p = plain.sample_probs(logits, 0.7, top_k=5)
    assert ((p > 0).sum(-1) == 5).all()
    assert torch.allclose(p.sum(-1), torch.ones(3))
    # ties at the k-th value are kept
    t = torch.tensor([[3.0, 2.0, 2.0, 1.0]])
    assert (plain.sample_probs(t, 1.0, top_k=2) > 0).sum() == 3


def test_exponential_race_draws_from_softmax():
    torch.manual_seed(0)
    logits = torch.tensor([1.0, 0.0, -1.0, 2.0, 0.5])
    n = 40000
    q = torch.empty(n, 5).exponential_(1)
    draws = plain.sample_with_exponentials(logits.expand(n, 5), 0.7, q)
    freq = torch.bincount(draws, minlength=5).float()
    expect = torch.softmax(logits / 0.7, -1) * n
    chi2 = ((freq - expect) ** 2 / expect).sum().item()
    assert chi2 < 18.5  # 4 degrees of freedom, p = 0.001
