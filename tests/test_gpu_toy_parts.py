"""More toy parts defined here, in the test, and put together into an architecture of their own:
a feed-forward that routes every token to one of several experts, a position encoding with
frequencies of its own that rotates only a part of a head in half-split pairs, a norm that centres
before it scales, a block arrangement in which mixer and feed-forward read the same normed
input, one with norms before and behind either branch (six parts), and one that has a mixer and a
norm and nothing else.  None of them exists in the framework; they are registered, built from random weights and
stepped through the engine in portions and mixed batches, and compared with a plain whole-sequence
computation written here.  They are toys, not anybody's model."""

from dataclasses import dataclass
from typing import Dict, Tuple

import pytest
import torch
import torch.nn.functional as F

from . import schedules
from .helpers import random_tokens
from .plain import llama as plain
from .test_gpu_engine import run_trace

pytestmark = pytest.mark.gpu

HIDDEN, VOCAB, HEADS, KV, DH, ROT, FFN, EXPERTS, SANDWICH_SCALE, WIDE_PAGE = 48, 83, 6, 3, 16, 8, 40, 3, 0.5, 32


@dataclass(frozen=True)
class ToyConfig:
    eps: float = 1e-4


def toy_frequencies() -> torch.Tensor:
    return 0.7 / (1.0 + torch.arange(ROT // 2, dtype=torch.float32)) ** 2


def _register():
    from torchllms_amd.config import ArchSpec, register_architecture
    from torchllms_amd.config.spec import LayerRun, LayerSpec, ModelSpec, PartSpec, standard_layer
    from torchllms_amd.parts import BLOCKS, FEED_FORWARDS, NORMS, POSITIONS, Block, FeedForward, Norm, ParamSpec, PositionEncoding
    from torchllms_amd.parts.positions import RotaryArgs
    from torchllms_amd.weights import NameRule

    if "toy_routed" not in FEED_FORWARDS:

        @FEED_FORWARDS.register("toy_routed")
        class RoutedFeedForward(FeedForward):
            """Every token goes to the expert with the largest router logit (32-bit logits, lowest
            index on ties) and comes back scaled by the sigmoid of that logit."""

            def __init__(self, hidden_size, intermediate_size, experts):
                self.hidden_size, self.intermediate_size, self.experts = hidden_size, intermediate_size, experts

            def param_specs(self):
                out = {"router.weight": ParamSpec((self.experts, self.hidden_size))}
                for e in range(self.experts):
                    out[f"experts.{e}.up.weight"] = ParamSpec((self.intermediate_size, self.hidden_size))
                    out[f"experts.{e}.down.weight"] = ParamSpec((self.hidden_size, self.intermediate_size))
                return out

            def bind(self, tensors):
                self.router = tensors["router.weight"]
                self.up = [tensors[f"experts.{e}.up.weight"] for e in range(self.experts)]
                self.down = [tensors[f"experts.{e}.down.weight"] for e in range(self.experts)]

            def forward(self, x, ctx):
                logits = F.linear(x.float(), self.router.float())
                best, chosen = logits.max(dim=-1)
                out = torch.zeros_like(x)
                for e in range(self.experts):
                    rows = (chosen == e).nonzero().flatten()
                    if rows.numel():
                        y = F.linear(F.gelu(F.linear(x[rows], self.up[e])), self.down[e])
                        out[rows] = (y.float() * torch.sigmoid(best[rows, None])).to(x.dtype)
                return out

        @POSITIONS.register("toy_partial_rotary")
        class PartialRotary(PositionEncoding):
            """The first ``rotary_dim`` channels of a head rotate, channel i with i + rotary_dim/2,
            by position times frequencies that follow no power law; the rest of the head passes."""

            def __init__(self, rotary_dim):
                self.rotary_dim = rotary_dim
                self.args = None

            def to(self, device):
                self.args = RotaryArgs(toy_frequencies().to(device), self.rotary_dim, 1)

            def rotary_args(self):
                return self.args

        @NORMS.register("toy_centred")
        class CentredNorm(Norm):
            """(x - mean) / sqrt(var + eps) * weight + bias, in 32-bit, with the framework's default
            ways of adding the residual and of picking rows."""

            def __init__(self, size, eps):
                self.size, self.eps = size, eps

            def param_specs(self):
                return {"weight": ParamSpec((self.size,), kind="vector", init="ones"), "bias": ParamSpec((self.size,), kind="vector", init="zeros")}

            def bind(self, tensors):
                self.weight, self.bias = tensors["weight"], tensors["bias"]

            def forward(self, x):
                return F.layer_norm(x.float(), (self.size,), self.weight.float(), self.bias.float(), self.eps).to(x.dtype)

        @BLOCKS.register("toy_parallel")
        class ParallelBlock(Block):
            """``out = x + mixer(norm(x)) + ffn(norm(x))``: one norm (the mixer's), both branches read it."""

            SLOTS = {"mixer_norm": "norm", "mixer": "mixer", "ffn": "feed_forward"}

            def forward(self, h, delta, ctx, cache):
                from torchllms_amd.kernels import ops

                h, y = self.mixer_norm.forward_add(h, self.mixer_norm.delta(delta))
                # (a branch may come back as the unadded sums of a split product: see ops.SplitSums)
                return h, ops.resolved(self.mixer.forward(y, ctx, cache["mixer"])) + ops.resolved(self.ffn.forward(y, ctx))

        @BLOCKS.register("toy_sandwich")
        class SandwichBlock(Block):
            """``h = x + scale * post_a(mixer(pre_a(x))); out = h + scale * post_f(ffn(pre_f(h)))``: four
            norms in a layer, and a constant of the arrangement's own."""

            SLOTS = {"pre_a": "norm", "mixer": "mixer", "post_a": "norm", "pre_f": "norm", "ffn": "feed_forward", "post_f": "norm"}

            def __init__(self, parts, scale):
                super().__init__(parts)
                self.scale = scale

            def forward(self, h, delta, ctx, cache):
                from torchllms_amd.kernels import ops

                h, y = self.pre_a.forward_add(h, self.pre_a.delta(delta))
                a = self.post_a.forward(ops.resolved(self.mixer.forward(y, ctx, cache["mixer"]))) * self.scale
                h, y = self.pre_f.forward_add(h, a)
                return h, self.post_f.forward(ops.resolved(self.ffn.forward(y, ctx))) * self.scale

        @BLOCKS.register("toy_mixer_only")
        class MixerOnlyBlock(Block):
            """``out = x + mixer(norm(x))``: a layer without a feed-forward."""

            SLOTS = {"norm": "norm", "mixer": "mixer"}

            def forward(self, h, delta, ctx, cache):
                h, y = self.norm.forward_add(h, self.norm.delta(delta))
                return h, self.mixer.forward(y, ctx, cache["mixer"])

    def spec(cfg: ToyConfig) -> ModelSpec:
        rope = PartSpec("toy_partial_rotary", dict(rotary_dim=ROT))
        centred = PartSpec("toy_centred", dict(size=HIDDEN, eps=cfg.eps))
        rms = PartSpec("rmsnorm", dict(size=HIDDEN, eps=cfg.eps))
        routed = PartSpec("toy_routed", dict(hidden_size=HIDDEN, intermediate_size=FFN, experts=EXPERTS))
        dense = PartSpec("swiglu", dict(hidden_size=HIDDEN, intermediate_size=FFN))
        attn = PartSpec("attention", dict(hidden_size=HIDDEN, num_heads=HEADS, num_kv_heads=KV, head_dim=DH, qkv_bias=False,
                                          softmax_scale=DH ** -0.5, window=0, position=rope))
        # the last layer's keys and values lie in pages of another size than the engine's
        attn_wide_pages = PartSpec("attention", dict(attn.params, kv_page_size=WIDE_PAGE))
        layers = [
            standard_layer("layers.0", "pre_norm", attn, routed, centred, rms),
            LayerSpec("layers.1", "toy_parallel", {"mixer_norm": centred, "mixer": attn, "ffn": dense}),
            standard_layer("layers.2", "pre_norm", attn, routed, rms, centred),
            LayerSpec("layers.3", "toy_sandwich", {"pre_a": rms, "mixer": attn, "post_a": centred, "pre_f": centred, "ffn": dense,
                                                   "post_f": rms}, {"scale": SANDWICH_SCALE}),
            LayerSpec("layers.4", "toy_mixer_only", {"norm": rms, "mixer": attn_wide_pages}),
        ]
        return ModelSpec("ToyRoutedForCausalLM", HIDDEN, VOCAB, 512, PartSpec("embedding", dict(vocab_size=VOCAB, hidden_size=HIDDEN)),
                         layers, [LayerRun(i) for i in range(5)], centred,
                         PartSpec("lm_head", dict(vocab_size=VOCAB, hidden_size=HIDDEN, tied=False)))

    def rules(cfg):
        names = ["embed.weight", "final_norm.weight", "final_norm.bias", "head.weight"]
        per_layer = ["mixer_norm.weight", "mixer_norm.bias", "ffn_norm.weight", "ffn_norm.bias", "ffn.w1.weight", "ffn.w2.weight",
                     "ffn.w3.weight", "ffn.router.weight", "mixer.wq.weight", "mixer.wk.weight", "mixer.wv.weight", "mixer.wo.weight",
                     "norm.weight"]
        per_layer += [f"{slot}.{t}" for slot in ("pre_a", "post_a", "pre_f", "post_f") for t in ("weight", "bias")]
        per_layer += [f"ffn.experts.{e}.{m}.weight" for e in range(EXPERTS) for m in ("up", "down")]
        return [NameRule(n, n) for n in names] + [NameRule("layers.{}." + n, "layers.{}." + n) for n in per_layer]

    return register_architecture(ArchSpec("ToyRoutedForCausalLM", lambda d: ToyConfig(**{k: v for k, v in d.items() if k != "architectures"}), spec, rules))


def plain_toy(w: Dict[str, torch.Tensor], cfg: ToyConfig, tokens):
    """The same model over a whole sequence, no cache, no engine."""
    S = len(tokens)
    ang = torch.arange(S, dtype=torch.float32)[:, None] * toy_frequencies()[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]

    def rotate(x):  # [S, heads, DH]: channel i pairs with i + ROT / 2 among the first ROT channels
        a, b, rest = x[..., : ROT // 2], x[..., ROT // 2 : ROT], x[..., ROT:]
        return torch.cat([a * cos - b * sin, b * cos + a * sin, rest], dim=-1)

    def centred(x, p):
        return F.layer_norm(x, (HIDDEN,), w[p + "weight"], w[p + "bias"], cfg.eps)

    def norm(layer, which, x):
        p = f"layers.{layer}.{which}."
        return centred(x, p) if p + "bias" in w else plain.rms_norm(x, w[p + "weight"], cfg.eps)

    def attn(layer, x):
        p = f"layers.{layer}.mixer."
        q = rotate(F.linear(x, w[p + "wq.weight"]).view(S, HEADS, DH))
        k = rotate(F.linear(x, w[p + "wk.weight"]).view(S, KV, DH))
        v = F.linear(x, w[p + "wv.weight"]).view(S, KV, DH)
        rows = [plain.attention(q[i : i + 1], k[: i + 1], v[: i + 1]) for i in range(S)]
        return F.linear(torch.cat(rows), w[p + "wo.weight"])

    def routed(layer, x):
        p = f"layers.{layer}.ffn."
        logits = F.linear(x, w[p + "router.weight"])
        out = []
        for t in range(S):
            e = int(logits[t].argmax())
            y = F.linear(F.gelu(F.linear(x[t], w[p + f"experts.{e}.up.weight"])), w[p + f"experts.{e}.down.weight"])
            out.append(y * torch.sigmoid(logits[t, e]))
        return torch.stack(out)

    def dense(layer, x):
        p = f"layers.{layer}.ffn."
        return plain.swiglu(x, w[p + "w1.weight"], w[p + "w3.weight"], w[p + "w2.weight"])

    h = w["embed.weight"][torch.tensor(tokens)]
    h = h + attn(0, norm(0, "mixer_norm", h))
    h = h + routed(0, norm(0, "ffn_norm", h))
    y = norm(1, "mixer_norm", h)
    h = h + attn(1, y) + dense(1, y)
    h = h + attn(2, norm(2, "mixer_norm", h))
    h = h + routed(2, norm(2, "ffn_norm", h))
    h = h + SANDWICH_SCALE * norm(3, "post_a", attn(3, norm(3, "pre_a", h)))
    h = h + SANDWICH_SCALE * norm(3, "post_f", dense(3, norm(3, "pre_f", h)))
    h = h + attn(4, norm(4, "norm", h))
    return F.linear(centred(h, "final_norm."), w["head.weight"])


def test_toy_parts_are_registered_built_and_stepped():
    from torchllms_amd.config.spec import LayerRun, LayerSpec, ModelSpec
    from torchllms_amd.engine import Engine
    from torchllms_amd.parts import Model
    from torchllms_amd.weights import random_tensors

    arch = _register()
    cfg = ToyConfig()
    expected = Model(arch.model_spec(cfg)).param_specs()
    # only what each layer's parts declare: no router in the dense layer, no bias under an RMS norm
    assert "layers.1.ffn.router.weight" not in expected and "layers.0.ffn.router.weight" in expected
    assert "layers.0.ffn_norm.bias" not in expected and "layers.0.mixer_norm.bias" in expected
    # the arrangement decides which parts a layer has: one norm in the parallel layer, four in the sandwich,
    # no feed-forward in the last
    assert not any(n.startswith("layers.1.ffn_norm") for n in expected)
    assert {n.split(".")[2] for n in expected if n.startswith("layers.3.")} == {"pre_a", "mixer", "post_a", "pre_f", "ffn", "post_f"}
    assert {n.split(".")[2] for n in expected if n.startswith("layers.4.")} == {"norm", "mixer"}
    with pytest.raises(ValueError, match="lacks \\['ffn'\\]"):
        Model(ModelSpec("x", HIDDEN, VOCAB, 8, arch.model_spec(cfg).embedding,
                        [LayerSpec("layers.0", "toy_parallel", {"mixer_norm": arch.model_spec(cfg).final_norm,
                                                                "mixer": arch.model_spec(cfg).layers[0].parts["mixer"]})],
                        [LayerRun(0)], arch.model_spec(cfg).final_norm, arch.model_spec(cfg).head))
    w = random_tensors(expected, seed=11, dtype=torch.float32, norm_jitter=0.2)
    for name in w:
        if name.endswith(("wq.weight", "wk.weight")):
            w[name] = w[name] * 15  # sharper attention than N(0, 0.02) gives
        if name.endswith("router.weight"):
            w[name] = w[name] * 40  # clear decisions: a near tie would turn rounding into another expert
        if name.endswith("bias"):
            w[name] = torch.randn_like(w[name]) * 0.1
    requests = {f"t{i}": random_tokens(n, VOCAB, 700 + i) for i, n in enumerate([37, 64, 21, 50])}
    truth = {rid: plain_toy(w, cfg, t) for rid, t in requests.items()}
    # every expert is used, so the routing is real
    x = plain.rms_norm(w["embed.weight"][torch.tensor(requests["t1"])], torch.ones(HIDDEN), cfg.eps)
    assert len(set(F.linear(x, w["layers.0.ffn.router.weight"]).argmax(-1).tolist())) == EXPERTS
    traces = {"whole": schedules.whole(requests), "portions": schedules.portions(requests), "mixed": schedules.mixed(requests)}
    pool_tokens = max(schedules.max_live_tokens(t) for t in traces.values())
    eng = Engine(arch, cfg, {k: v.to("cuda:0") for k, v in w.items()}, torch.float32, page_size=4,
                 num_pages=-(-pool_tokens // 4), max_seqs=4, max_model_len=512)
    # two groups of pages: the engine's page size for four layers, the last layer's own; both hold the same tokens
    assert [(g.page_size, g.run_ids) for g in eng.cache.groups] == [(0, tuple((i, "mixer") for i in range(4))), (WIDE_PAGE, ((4, "mixer"),))]
    assert eng.cache.page_sizes == [4, WIDE_PAGE] and not eng.cache.states
    assert eng.cache.pools[1].num_pages == -(-eng.cache.pools[0].num_pages * 4 // WIDE_PAGE)
    assert eng.graphs is None  # no part here says graph_safe: the routed feed-forward's launches depend on the tokens
    for name, steps in traces.items():
        got = run_trace(eng, steps)
        for (rid, pos), row in got.items():
            assert (row - truth[rid][pos]).abs().max().item() < 5e-5, f"{name}: {rid} position {pos}"


def test_toy_parts_in_bfloat16_stay_near_the_plain_model():
    """The same architecture in bfloat16 through the fast kernels (MFMA attention with the toy
    rotation fused into the projection): as near to the 32-bit truth as bfloat16 allows."""
    from torchllms_amd.engine import Engine
    from torchllms_amd.parts import Model
    from torchllms_amd.weights import random_tensors

    arch = _register()
    cfg = ToyConfig()
    w = random_tensors(Model(arch.model_spec(cfg)).param_specs(), seed=12, dtype=torch.float32, norm_jitter=0.2)
    for name in w:
        if name.endswith("router.weight"):
            w[name] = w[name] * 40
        w[name] = w[name].bfloat16().float()
    requests = {f"b{i}": random_tokens(n, VOCAB, 800 + i) for i, n in enumerate([30, 45])}
    truth = {rid: plain_toy(w, cfg, t) for rid, t in requests.items()}
    steps = schedules.portions(requests)
    eng = Engine(arch, cfg, {k: v.to("cuda:0").bfloat16() for k, v in w.items()}, torch.bfloat16, page_size=16,
                 num_pages=16, max_seqs=4, max_model_len=512)
    got = run_trace(eng, steps)
    worst = max((row - truth[rid][pos]).abs().max().item() for (rid, pos), row in got.items())
    scale = max(t.abs().max().item() for t in truth.values())
    assert worst < 0.06 * scale, (worst, scale)


def test_a_toy_feed_forward_may_take_normed_rows_and_make_a_tensor_of_them():
    """A part that says ``takes_normed_rows`` is handed the norm's rows with their statistics not yet
    applied on bfloat16 steps of few rows; ``ops.resolved`` makes the normed tensor of them, the very
    bits that the same part gets when it does not say so (the product before the norm adds itself to
    the residual rows with the roundings of the norm kernel, which then runs on its result)."""
    from torchllms_amd.config.spec import PartSpec
    from torchllms_amd.kernels import ops
    from torchllms_amd.parts import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, FeedForward, ParamSpec
    from .test_gpu_parts import _ctx_and_cache, _step

    seen = []

    class Doubling(FeedForward):
        graph_safe = True

        def __init__(self, hidden_size):
            self.hidden_size = hidden_size

        def param_specs(self):
            return {"w.weight": ParamSpec((self.hidden_size, self.hidden_size))}

        def bind(self, tensors):
            self.w = tensors["w.weight"]

        def forward(self, x, ctx):
            seen.append(type(x).__name__)
            return ops.linear(ops.resolved(x), self.w) * 2

    class DoublingThatTakesThem(Doubling):
        takes_normed_rows = True

    FEED_FORWARDS["toy_doubling"], FEED_FORWARDS["toy_doubling_takes"] = Doubling, DoublingThatTakesThem
    try:
        torch.manual_seed(3)
        D, S = 64, 6
        outs = []
        for kind in ("toy_doubling", "toy_doubling_takes"):
            block = BLOCKS["pre_norm"]({
                "mixer": MIXERS.build(PartSpec("attention", dict(hidden_size=D, num_heads=4, num_kv_heads=2, head_dim=16, qkv_bias=False,
                                                                 softmax_scale=0.25, window=0,
                                                                 position=PartSpec("rope", dict(head_dim=16, rotary_dim=16, theta=1e4, scaling=None))))),
                "ffn": FEED_FORWARDS.build(PartSpec(kind, dict(hidden_size=D))),
                "mixer_norm": NORMS.build(PartSpec("rmsnorm", dict(size=D, eps=1e-5))),
                "ffn_norm": NORMS.build(PartSpec("rmsnorm", dict(size=D, eps=1e-5))),
            })
            gen = torch.Generator().manual_seed(5)
            w = {n: ((torch.randn(s.shape, generator=gen) * 0.2) if s.init == "normal" else (0.5 + torch.rand(s.shape, generator=gen))).bfloat16()
                 for n, s in block.param_specs().items()}
            block.bind({k: v.to("cuda:0") for k, v in w.items()})
            x = (torch.randn(S, D, generator=torch.Generator().manual_seed(6)) * 2).bfloat16().to("cuda:0")
            cache = _ctx_and_cache(S, 2, 16, 4, torch.bfloat16)
            h, delta = block.forward(x, None, _step(cache, "r", S), {"mixer": cache.kv_view(0)})
            outs.append((h, ops.resolved(delta)))
        assert seen == ["Tensor", "NormedRows"]
        assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    finally:
        del FEED_FORWARDS["toy_doubling"], FEED_FORWARDS["toy_doubling_takes"]
