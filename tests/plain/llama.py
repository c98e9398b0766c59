"""A plain, slow implementation of the Llama 3 dense decoder: whole sequences, no cache, one
function per part, only ``torch`` tensor arithmetic.  It shares no code with ``torchllms_amd``.

It is written from the formulas of the reference (every function cites the reference's file:line),
which was read, not run.  Tests compare the engine against it.

Conventions: one sequence at a time; activations are [S, ...]; ``weights`` is the dict of a
checkpoint's tensors under the checkpoint's own names (``model.layers.0.self_attn.q_proj.weight``),
whose q/k rows are laid out for half-split rotary pairs.  ``forward`` first brings q/k rows into the
interleaved layout the reference computes in.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch
import torch.nn.functional as F


# ----------------------------------------------------------------------------- norm
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """reference: torchllms/models/networks.py:195-200.
    Statistics in float32; eps inside the root, added to the mean of squares; the result is cast
    back to x's dtype *before* the multiply with the weight."""
    xf = x.float()
    normed = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return normed.type_as(x) * weight


# ----------------------------------------------------------------------------- rotary positions
def rope_inverse_frequencies(head_dim: int, theta: float, scaling: Optional[dict]) -> torch.Tensor:
    """reference: torchllms/models/networks.py:252-279.
    float32 throughout.  ``scaling`` None or rope_type "default": plain geometric progression.
    rope_type "llama3": long wavelengths divided by factor, a linear blend in the middle band."""
    freqs = 1.0 / (theta ** (torch.arange(0, head_dim, 2)[: head_dim // 2].float() / head_dim))
    if scaling is None or scaling.get("rope_type", "default") == "default":
        return freqs
    if scaling["rope_type"] != "llama3":
        raise ValueError(f"Unknown RoPE type: {scaling['rope_type']}")
    factor = scaling["factor"]
    lo_f = scaling["low_freq_factor"]
    hi_f = scaling["high_freq_factor"]
    old_len = scaling["original_max_position_embeddings"]
    low_freq_wavelen = old_len / lo_f
    high_freq_wavelen = old_len / hi_f
    out = []
    # element by element, the way the formula reads
    for f in freqs:
        wavelen = 2 * math.pi / f
        if wavelen > low_freq_wavelen:
            f_new = f / factor
        else:
            f_new = f
        if not (wavelen < high_freq_wavelen) and not (wavelen > low_freq_wavelen):
            smooth = (old_len / wavelen - lo_f) / (hi_f - lo_f)
            f_new = (1 - smooth) * f_new / factor + smooth * f_new
        out.append(f_new)
    return torch.stack(out).float()


def rope_angles(positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """reference: torchllms/models/networks.py:284-297.  Outer product of float32 positions and
    float32 inverse frequencies: [S, head_dim/2]."""
    return torch.outer(positions.float(), inv_freq.float()).float()


def rope_rotate_interleaved(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """reference: torchllms/models/networks.py:332-352.
    x [S, H, dh]; pair i is (x[..., 2i], x[..., 2i+1]); float32 arithmetic, cast back at the end."""
    ang = rope_angles(positions, inv_freq)  # [S, dh/2]
    cos = ang.cos()[:, None, :]
    sin = ang.sin()[:, None, :]
    xf = x.float()
    even = xf[..., 0::2]
    odd = xf[..., 1::2]
    out = torch.empty_like(xf)
    out[..., 0::2] = even * cos - odd * sin
    out[..., 1::2] = odd * cos + even * sin
    return out.type_as(x)


def rope_rotate_half_split(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """The checkpoint's own convention, pair i = (x[..., i], x[..., i + dh/2]).  Not used by
    ``forward``; it pins the row permutation below (reference: checkpoint_converter.py:96-108 says
    the permutation exists "to account for different RoPE dimension orderings")."""
    ang = rope_angles(positions, inv_freq)
    cos = ang.cos()[:, None, :]
    sin = ang.sin()[:, None, :]
    xf = x.float()
    half = x.shape[-1] // 2
    a, b = xf[..., :half], xf[..., half:]
    return torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1).type_as(x)


def permute_rows_for_interleaved(w: torch.Tensor, n_heads: int, head_dim: int) -> torch.Tensor:
    """reference: torchllms/models/checkpoint_converter.py:96-108.
    Rows of a q/k projection [H * dh, D] (or a bias [H * dh]): within every head the row at
    offset i of the first half goes to 2i, the row at offset i of the second half to 2i + 1."""
    out = torch.empty_like(w)
    half = head_dim // 2
    for h in range(n_heads):
        base = h * head_dim
        for i in range(half):
            out[base + 2 * i] = w[base + i]
            out[base + 2 * i + 1] = w[base + half + i]
    return out


# ----------------------------------------------------------------------------- attention
def causal_mask(q_len: int, kv_len: int, dtype: torch.dtype) -> torch.Tensor:
    """reference: torchllms/models/utils.py:263-285.  mask[i, j] = 0 where key j is visible to
    query i (j <= i + kv_len - q_len), else the most negative finite value of the dtype."""
    past = kv_len - q_len
    mask = torch.full((q_len, kv_len), torch.finfo(dtype).min, dtype=dtype)
    for i in range(q_len):
        mask[i, : past + i + 1] = 0
    return mask


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: Optional[float] = None) -> torch.Tensor:
    """reference: torchllms/models/networks.py:355-397 (the eager formula).
    q [Sq, Hq, dh]; k, v [Sk, Hkv, dh] with Sk >= Sq (the last Sq keys belong to the queries).
    Query head h reads kv head h // (Hq / Hkv).  Returns [Sq, Hq * dh]."""
    sq, hq, dh = q.shape
    sk, hkv, _ = k.shape
    rep = hq // hkv
    qh = q.transpose(0, 1)  # [Hq, Sq, dh]
    kh = k.transpose(0, 1).repeat_interleave(rep, dim=0)
    vh = v.transpose(0, 1).repeat_interleave(rep, dim=0)
    if scale is None:
        scores = torch.matmul(qh, kh.transpose(1, 2)) / math.sqrt(dh)
    else:
        scores = torch.matmul(qh, kh.transpose(1, 2)) * scale
    scores = scores + causal_mask(sq, sk, q.dtype).to(q.device)
    weights = F.softmax(scores, dim=-1)
    out = torch.matmul(weights, vh)  # [Hq, Sq, dh]
    return out.transpose(0, 1).reshape(sq, hq * dh)


# ----------------------------------------------------------------------------- feed-forward
def swiglu(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """reference: torchllms/models/networks.py:592-605.  w2(silu(w1 x) * w3 x), no biases."""
    return F.linear(F.silu(F.linear(x, w_gate)) * F.linear(x, w_up), w_down)


# ----------------------------------------------------------------------------- whole model
def layer_weights(weights: Dict[str, torch.Tensor], i: int, cfg: dict) -> Dict[str, torch.Tensor]:
    hq = cfg["num_attention_heads"]
    hkv = cfg.get("num_key_value_heads") or hq
    dh = cfg.get("head_dim") or cfg["hidden_size"] // hq
    p = f"model.layers.{i}."
    out = {
        "wq": permute_rows_for_interleaved(weights[p + "self_attn.q_proj.weight"], hq, dh),
        "wk": permute_rows_for_interleaved(weights[p + "self_attn.k_proj.weight"], hkv, dh),
        "wv": weights[p + "self_attn.v_proj.weight"],
        "wo": weights[p + "self_attn.o_proj.weight"],
        "w1": weights[p + "mlp.gate_proj.weight"],
        "w3": weights[p + "mlp.up_proj.weight"],
        "w2": weights[p + "mlp.down_proj.weight"],
        "attention_norm": weights[p + "input_layernorm.weight"],
        "ffn_norm": weights[p + "post_attention_layernorm.weight"],
    }
    if cfg.get("attention_bias", False):
        out["bq"] = permute_rows_for_interleaved(weights[p + "self_attn.q_proj.bias"], hq, dh)
        out["bk"] = permute_rows_for_interleaved(weights[p + "self_attn.k_proj.bias"], hkv, dh)
        out["bv"] = weights[p + "self_attn.v_proj.bias"]
    return out


def attention_part(x: torch.Tensor, lw: Dict[str, torch.Tensor], cfg: dict, positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """reference: torchllms/models/networks.py:512-535,558 (projections, view into heads, rotary on
    q and k, attention, output projection)."""
    hq = cfg["num_attention_heads"]
    hkv = cfg.get("num_key_value_heads") or hq
    dh = cfg.get("head_dim") or cfg["hidden_size"] // hq
    s = x.shape[0]
    q = F.linear(x, lw["wq"], lw.get("bq")).view(s, hq, dh)
    k = F.linear(x, lw["wk"], lw.get("bk")).view(s, hkv, dh)
    v = F.linear(x, lw["wv"], lw.get("bv")).view(s, hkv, dh)
    q = rope_rotate_interleaved(q, positions, inv_freq)
    k = rope_rotate_interleaved(k, positions, inv_freq)
    return F.linear(attention(q, k, v), lw["wo"])


def block(x: torch.Tensor, lw: Dict[str, torch.Tensor], cfg: dict, positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """reference: torchllms/models/networks.py:635-644.  Pre-norm residual block."""
    eps = cfg.get("rms_norm_eps") or 1e-5
    h = x + attention_part(rms_norm(x, lw["attention_norm"], eps), lw, cfg, positions, inv_freq)
    return h + swiglu(rms_norm(h, lw["ffn_norm"], eps), lw["w1"], lw["w3"], lw["w2"])


def forward(weights: Dict[str, torch.Tensor], cfg: dict, tokens: List[int], dtype: torch.dtype = torch.float32,
            start_position: int = 0, device: str = "cpu") -> torch.Tensor:
    """reference: torchllms/models/networks.py:1017-1047.  Embedding, blocks, final norm, output
    matrix (the embedding matrix when ``tie_word_embeddings``).  Returns logits [S, V] in ``dtype``.
    ``start_position`` shifts all positions (only distances may matter).  ``device``: where torch
    does the arithmetic (the same tensor operations anywhere)."""
    w = {k: v.to(device=device, dtype=dtype) for k, v in weights.items()}
    hq = cfg["num_attention_heads"]
    dh = cfg.get("head_dim") or cfg["hidden_size"] // hq
    theta = cfg.get("rope_theta") or 10000.0
    inv_freq = rope_inverse_frequencies(dh, theta, cfg.get("rope_scaling"))
    inv_freq = inv_freq.to(device)
    ids = torch.tensor(tokens, dtype=torch.long, device=device)
    positions = torch.arange(start_position, start_position + len(tokens), device=device)
    h = w["model.embed_tokens.weight"][ids]
    for i in range(cfg["num_hidden_layers"]):
        h = block(h, layer_weights(w, i, cfg), cfg, positions, inv_freq)
    eps = cfg.get("rms_norm_eps") or 1e-5
    h = rms_norm(h, w["model.norm.weight"], eps)
    out_w = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return F.linear(h, out_w)


# ----------------------------------------------------------------------------- sampling
def sample_probs(logits: torch.Tensor, temperature: float, top_k: Optional[int] = None) -> torch.Tensor:
    """reference: torchllms/inference/utils.py:25-33.  logits / max(T, 1e-5); with top_k everything
    below the k-th largest becomes -inf (ties kept); softmax."""
    x = logits / max(temperature, 1e-5)
    if top_k is not None:
        kth = torch.sort(x, dim=-1, descending=True).values[..., min(top_k, x.shape[-1]) - 1]
        x = torch.where(x < kth.unsqueeze(-1), torch.full_like(x, float("-inf")), x)
    return F.softmax(x, dim=-1)


def sample_with_exponentials(logits: torch.Tensor, temperature: float, q: torch.Tensor, top_k: Optional[int] = None) -> torch.Tensor:
    """reference: torchllms/inference/utils.py:18-22,36-48.  Greedy at temperature 0; otherwise
    argmax(probs / q) with q ~ Exponential(1) given by the caller."""
    if temperature == 0:
        return torch.argmax(logits, dim=-1)
    return torch.argmax(sample_probs(logits, temperature, top_k) / q, dim=-1)
