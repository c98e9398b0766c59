"""A toy architecture defined here, in the test: a mixer with state of its own beside attention
layers (one of them windowed), an execution order that runs a layer twice and lets a run read
another run's cache.  It is registered, built from random weights and stepped through the engine
in portions and mixed batches without any change to the framework's files, and compared with a
plain whole-sequence computation written here."""

import json
from dataclasses import dataclass
from typing import Dict

import pytest
import torch
import torch.nn.functional as F

from . import schedules
from .helpers import random_tokens, read_folder
from .plain import llama as plain
from .test_gpu_engine import run_trace

pytestmark = pytest.mark.gpu

HIDDEN, STATE, VOCAB, HEADS, KV, DH, FFN, WINDOW, WINDOW_PAGE = 40, 24, 97, 4, 2, 16, 56, 6, 8


@dataclass(frozen=True)
class ToyConfig:
    """(Nothing but what the toy models need: no ``architectures``, no end-of-sequence id, none of the
    attributes of the framework's own configuration.)"""

    decay: float = 0.8
    end_token: int = -1  # the token id that ends a generation, if any


def _config_from_dict(d):
    return ToyConfig(**{k: v for k, v in d.items() if k != "architectures"})


def _register():
    from torchllms_amd.config import ArchSpec, register_architecture
    from torchllms_amd.config.spec import LayerRun, ModelSpec, PartSpec, standard_layer
    from torchllms_amd.parts import MIXERS, Mixer, ParamSpec, StateNeed
    from torchllms_amd.weights import NameRule

    if "toy_decay" not in MIXERS:

        @MIXERS.register("toy_decay")
        class DecayMixer(Mixer):
            """s_t = decay * s_{t-1} + W_in x_t ;  y_t = W_out s_t.  The state s lives in the
            request's slot, so it carries over from one step to the next."""

            def __init__(self, hidden_size, state_size, decay):
                self.hidden_size, self.state_size, self.decay = hidden_size, state_size, decay

            def param_specs(self):
                return {"w_in.weight": ParamSpec((self.state_size, self.hidden_size)),
                        "w_out.weight": ParamSpec((self.hidden_size, self.state_size))}

            def cache_need(self):
                return StateNeed(shape=(self.state_size,), dtype="float32")

            def bind(self, tensors):
                self.w_in, self.w_out = tensors["w_in.weight"], tensors["w_out.weight"]

            def forward(self, x, ctx, cache):
                u = F.linear(x.float(), self.w_in.float())
                states = torch.empty_like(u)
                lay = ctx.host
                for row in range(lay.n_seqs):
                    s = cache.tensor[int(lay.slot_ids[row])]
                    for t in range(int(lay.qo_indptr[row]), int(lay.qo_indptr[row + 1])):
                        s.mul_(self.decay).add_(u[t])
                        states[t] = s
                return F.linear(states, self.w_out.float()).to(x.dtype)

    def spec(cfg: ToyConfig) -> ModelSpec:
        rope = PartSpec("rope", dict(head_dim=DH, rotary_dim=DH, theta=100.0, scaling=None))
        norm = PartSpec("rmsnorm", dict(size=HIDDEN, eps=1e-5))
        ffn = PartSpec("swiglu", dict(hidden_size=HIDDEN, intermediate_size=FFN))

        def attn(window):
            # the windowed layer keeps its keys in pages of 8 tokens, whatever the engine's page size
            return PartSpec("attention", dict(hidden_size=HIDDEN, num_heads=HEADS, num_kv_heads=KV, head_dim=DH, qkv_bias=False,
                                              softmax_scale=DH ** -0.5, window=window, position=rope,
                                              kv_page_size=WINDOW_PAGE if window else None))

        mixers = [attn(0), PartSpec("toy_decay", dict(hidden_size=HIDDEN, state_size=STATE, decay=cfg.decay)), attn(WINDOW)]
        layers = [standard_layer(f"layers.{i}", "pre_norm", m, ffn, norm, norm) for i, m in enumerate(mixers)]
        order = [LayerRun(0), LayerRun(1), LayerRun(2), LayerRun(1), LayerRun(0, cache_from=0)]
        return ModelSpec("ToyHybridForCausalLM", HIDDEN, VOCAB, 512, PartSpec("embedding", dict(vocab_size=VOCAB, hidden_size=HIDDEN)),
                         layers, order, norm, PartSpec("lm_head", dict(vocab_size=VOCAB, hidden_size=HIDDEN, tied=True)))

    def rules(cfg):
        names = ["embed.weight", "final_norm.weight"]
        per_layer = ["mixer_norm.weight", "ffn_norm.weight", "ffn.w1.weight", "ffn.w2.weight", "ffn.w3.weight",
                     "mixer.wq.weight", "mixer.wk.weight", "mixer.wv.weight", "mixer.wo.weight",
                     "mixer.w_in.weight", "mixer.w_out.weight"]
        return [NameRule(n, n) for n in names] + [NameRule("layers.{}." + n, "layers.{}." + n) for n in per_layer]

    return register_architecture(ArchSpec("ToyHybridForCausalLM", _config_from_dict, spec, rules, stop_token_ids=lambda cfg: [cfg.end_token] if cfg.end_token >= 0 else []))


def plain_toy(w: Dict[str, torch.Tensor], cfg: ToyConfig, tokens):
    """The same model over a whole sequence, no cache, no engine."""
    S = len(tokens)
    pos = torch.arange(S)
    f = plain.rope_inverse_frequencies(DH, 100.0, None)
    h = w["embed.weight"][torch.tensor(tokens)]
    kept = {}

    def attn(run, layer, x, window, borrow=None):
        p = f"layers.{layer}.mixer."
        q = plain.rope_rotate_interleaved(F.linear(x, w[p + "wq.weight"]).view(S, HEADS, DH), pos, f)
        if borrow is None:
            k = plain.rope_rotate_interleaved(F.linear(x, w[p + "wk.weight"]).view(S, KV, DH), pos, f)
            v = F.linear(x, w[p + "wv.weight"]).view(S, KV, DH)
            kept[run] = (k, v)
        else:
            k, v = kept[borrow]
        rows = []
        for i in range(S):
            lo = max(i - window + 1, 0) if window else 0
            rows.append(plain.attention(q[i : i + 1], k[lo : i + 1], v[lo : i + 1]))
        return F.linear(torch.cat(rows), w[p + "wo.weight"])

    def decay(layer, x):
        p = f"layers.{layer}.mixer."
        u = F.linear(x, w[p + "w_in.weight"])
        s = torch.zeros(STATE)
        out = []
        for t in range(S):
            s = cfg.decay * s + u[t]
            out.append(s)
        return F.linear(torch.stack(out), w[p + "w_out.weight"])

    runs = [(0, None), (1, None), (2, None), (1, None), (0, 0)]
    for run, (layer, borrow) in enumerate(runs):
        p = f"layers.{layer}."
        x = plain.rms_norm(h, w[p + "mixer_norm.weight"], 1e-5)
        h = h + (decay(layer, x) if layer == 1 else attn(run, layer, x, WINDOW if layer == 2 else 0, borrow))
        h = h + plain.swiglu(plain.rms_norm(h, w[p + "ffn_norm.weight"], 1e-5), w[p + "ffn.w1.weight"], w[p + "ffn.w3.weight"], w[p + "ffn.w2.weight"])
    return F.linear(plain.rms_norm(h, w["final_norm.weight"], 1e-5), w["embed.weight"])


def test_toy_architecture_is_registered_built_and_stepped():
    from torchllms_amd.engine import Engine
    from torchllms_amd.parts import Model
    from torchllms_amd.weights import random_tensors

    arch = _register()
    cfg = ToyConfig()
    expected = Model(arch.model_spec(cfg)).param_specs()
    w = random_tensors(expected, seed=3, dtype=torch.float32, norm_jitter=0.1)
    for name in w:  # sharper attention and a livelier state than N(0, 0.02) gives
        if name.endswith(("wq.weight", "wk.weight")):
            w[name] = w[name] * 15
        if name.endswith(("w_in.weight", "w_out.weight")):
            w[name] = w[name] * 8
    requests = {f"t{i}": random_tokens(n, VOCAB, 500 + i) for i, n in enumerate([40, 70, 33, 55])}
    traces = {"whole": schedules.whole(requests), "portions": schedules.portions(requests), "mixed": schedules.mixed(requests)}
    pool_tokens = max(schedules.max_live_tokens(t) for t in traces.values())
    eng = Engine(arch, cfg, {k: v.to("cuda:0") for k, v in w.items()}, torch.float32, page_size=4,
                 num_pages=-(-pool_tokens // 4), max_seqs=4, max_model_len=512)
    # groups: full attention (runs 0 and the borrower's source), windowed attention in pages of another size,
    # and state slots for two runs; every group's pool holds the same number of tokens
    assert sorted((g.window, g.run_ids) for g in eng.cache.groups) == [(0, ((0, "mixer"),)), (WINDOW, ((2, "mixer"),))]
    assert eng.cache.page_sizes == [4, WINDOW_PAGE] and eng.cache.k_pages[1].shape[3] == WINDOW_PAGE
    assert eng.cache.pools[0].num_pages == -(-pool_tokens // 4) and eng.cache.pools[1].num_pages == -(-(-(-pool_tokens // 4) * 4) // WINDOW_PAGE)
    assert [(s.run_ids, s.shape) for s in eng.cache.states] == [(((1, "mixer"), (3, "mixer")), (STATE,))]
    truth = {rid: plain_toy(w, cfg, t) for rid, t in requests.items()}
    for name, steps in traces.items():
        got = run_trace(eng, steps)
        for (rid, pos), row in got.items():
            assert (row - truth[rid][pos]).abs().max().item() < 5e-5, f"{name}: {rid} position {pos}"
    # the windowed group gave pages back while requests were still running
    eng.admit("w")
    from torchllms_amd.engine import StepEntry

    eng.step([StepEntry("w", random_tokens(30, VOCAB, 9))])
    assert sum(p >= 0 for p in eng.cache.block_table("w", 1)) <= 2 < sum(p >= 0 for p in eng.cache.block_table("w", 0))
    assert len(eng.cache.block_table("w", 0)) == 8 and len(eng.cache.block_table("w", 1)) == 4  # 30 tokens in pages of 4 and of 8
    eng.free("w")


def test_toy_architecture_generates_through_the_host_path(tmp_path):
    """The same toy architecture from a model folder through ``LLM.generate``: the folder is written by
    the random-weights mode, config.json names the architecture, the scheduler and the sampling run as
    for any model, and generation stops on the token id that the architecture gives for its
    configuration.  Nothing on the way asks the configuration for what only the framework's own has."""
    from torchllms_amd.inference import LLM
    from torchllms_amd.weights import write_model_folder

    arch = _register()
    cfg = ToyConfig(decay=0.7)
    folder = write_model_folder(tmp_path / "toy", cfg, seed=4, dtype=torch.float32, norm_jitter=0.1, arch=arch)
    assert json.loads((folder / "config.json").read_text()) == {"decay": 0.7, "end_token": -1, "architectures": ["ToyHybridForCausalLM"]}
    _, w = read_folder(folder)
    prompts = [random_tokens(n, VOCAB, 40 + n) for n in (5, 23, 2)]
    kw = dict(precision="float32", max_len=200, max_bsz=2, page_size=4, max_num_batched_tokens=16)
    llm = LLM(str(folder), **kw)
    assert llm.eos_ids == [] and llm.engine.graphs is None  # (the toy mixer's launches depend on the plan)
    free = llm.generate(prompt_token_ids=prompts, max_new_tokens=30)
    for p, r in zip(prompts, free):
        toks = list(p)
        for _ in range(30):
            toks.append(int(plain_toy(w, cfg, toks)[-1].argmax()))
        assert r.token_ids == toks[len(p):] and r.stop_reason is None
    # the same weights with an end token in the configuration: one that the second request generates
    end = free[1].token_ids[7]
    folder = write_model_folder(tmp_path / "toy_end", ToyConfig(decay=0.7, end_token=end), seed=4, dtype=torch.float32, norm_jitter=0.1, arch=arch)
    llm = LLM(str(folder), **kw)
    assert llm.eos_ids == [end]
    stopped = llm.generate(prompt_token_ids=prompts, max_new_tokens=30)
    assert stopped[1].stop_reason == end and len(stopped[1].token_ids) <= 8
    for a, b in zip(free, stopped):
        cut = a.token_ids.index(end) + 1 if end in a.token_ids else 30
        assert b.token_ids == a.token_ids[:cut] and b.stop_reason == (end if end in a.token_ids else None)
    llm.engine.cache.check_invariants()
    assert llm.engine.cache.live == []


def _register_windowed():
    """Two attention layers from the framework's own parts, the second with a window of 20 keys in pages of
    8: every part is fit for a recorded graph, so decode steps of this model are replayed and prepared ahead."""
    from torchllms_amd.config import ArchSpec, register_architecture
    from torchllms_amd.config.spec import LayerRun, ModelSpec, PartSpec, standard_layer
    from torchllms_amd.weights import NameRule

    window = 20

    def spec(cfg: ToyConfig) -> ModelSpec:
        rope = PartSpec("rope", dict(head_dim=DH, rotary_dim=DH, theta=100.0, scaling=None))
        norm = PartSpec("rmsnorm", dict(size=HIDDEN, eps=1e-5))
        ffn = PartSpec("swiglu", dict(hidden_size=HIDDEN, intermediate_size=FFN))

        def attn(w):
            return PartSpec("attention", dict(hidden_size=HIDDEN, num_heads=HEADS, num_kv_heads=KV, head_dim=DH, qkv_bias=False,
                                              softmax_scale=DH ** -0.5, window=w, position=rope, kv_page_size=WINDOW_PAGE if w else None))

        layers = [standard_layer(f"layers.{i}", "pre_norm", attn(w), ffn, norm, norm) for i, w in enumerate([0, window])]
        return ModelSpec("ToyWindowedForCausalLM", HIDDEN, VOCAB, 512, PartSpec("embedding", dict(vocab_size=VOCAB, hidden_size=HIDDEN)),
                         layers, [LayerRun(0), LayerRun(1)], norm, PartSpec("lm_head", dict(vocab_size=VOCAB, hidden_size=HIDDEN, tied=True)))

    def rules(cfg):
        per_layer = ["mixer_norm.weight", "ffn_norm.weight", "ffn.w1.weight", "ffn.w2.weight", "ffn.w3.weight",
                     "mixer.wq.weight", "mixer.wk.weight", "mixer.wv.weight", "mixer.wo.weight"]
        return [NameRule(n, n) for n in ("embed.weight", "final_norm.weight")] + [NameRule("layers.{}." + n, "layers.{}." + n) for n in per_layer]

    arch = register_architecture(ArchSpec("ToyWindowedForCausalLM", _config_from_dict, spec, rules))
    return arch, window


def test_windowed_layers_decode_through_graphs_and_prepared_steps():
    """Decode steps of a model with a window are planned from the step before, replayed from a graph and
    prepared a step ahead like any other: the pages that the window gives back leave the plan's block tables
    as they leave the requests'.  Same bits as an engine that plans and launches every step by itself."""
    from torchllms_amd.engine import Engine, StepEntry
    from torchllms_amd.parts import Model
    from torchllms_amd.weights import random_tensors

    arch, window = _register_windowed()
    cfg = ToyConfig()
    w = random_tensors(Model(arch.model_spec(cfg)).param_specs(), seed=5, dtype=torch.float32, norm_jitter=0.1)
    for name in w:
        if name.endswith(("wq.weight", "wk.weight")):
            w[name] = w[name] * 15
    w = {k: v.to("cuda:0") for k, v in w.items()}
    make = lambda graphs: Engine(arch, cfg, w, torch.float32, page_size=4, num_pages=120, max_seqs=4, max_model_len=512, use_graphs=graphs)
    plain, ahead = make(False), make(True)
    toks = {r: random_tokens(200, VOCAB, 70 + i) for i, r in enumerate("abc")}
    start = {"a": 61, "b": 3, "c": 17}
    for eng in (plain, ahead):
        for r in toks:
            eng.admit(r)
        eng.step([StepEntry(r, toks[r][: start[r]], []) for r in toks])
    used, prepared = 0, None
    for step in range(90):
        entries = [StepEntry(r, [toks[r][start[r] + step]], [0]) for r in toks]
        plain._last_decode = None  # this engine plans every step from the requests' tables alone
        want = plain.step(entries)
        got = ahead.step_prepared(prepared, entries) if prepared is not None else None
        used += got is not None
        if got is None:
            got = ahead.step(entries)
        assert torch.equal(want, got), step
        prepared = ahead.prepare_decode()
        if prepared is not None:
            # the next step's plan names exactly the pages that the requests hold now
            for g in range(2):
                for row, r in enumerate("abc"):
                    table = ahead.cache.block_table(r, g)
                    assert prepared.layout.block_tables[g][row, : len(table)].tolist() == table, (step, g, r)
        ahead.cache.check_invariants()
    assert used >= 75  # all but the first steps of a shape, which run eagerly before they are recorded
    # the window gave pages back on the way: request a holds 151 tokens, of them the last 20 in the windowed group
    assert sum(p >= 0 for p in ahead.cache.block_table("a", 1)) <= -(-window // WINDOW_PAGE) + 1
    assert sum(p >= 0 for p in ahead.cache.block_table("a", 0)) == -(-151 // 4)
    got = ahead.step([StepEntry("a", [toks["a"][151]], [0]), StepEntry("b", [toks["b"][93]], []), StepEntry("c", [toks["c"][107]], [])])
    want = plain_windowed(w, toks["a"][:152], window)[-1]
    assert (got[0].cpu() - want).abs().max().item() < 5e-5


def plain_windowed(w, tokens, window):
    """The two-layer windowed model over a whole sequence, no cache, no engine."""
    w = {k: v.cpu() for k, v in w.items()}
    S = len(tokens)
    pos = torch.arange(S)
    f = plain.rope_inverse_frequencies(DH, 100.0, None)
    h = w["embed.weight"][torch.tensor(tokens)]
    for layer, win in enumerate([0, window]):
        p = f"layers.{layer}."
        x = plain.rms_norm(h, w[p + "mixer_norm.weight"], 1e-5)
        q = plain.rope_rotate_interleaved(F.linear(x, w[p + "mixer.wq.weight"]).view(S, HEADS, DH), pos, f)
        k = plain.rope_rotate_interleaved(F.linear(x, w[p + "mixer.wk.weight"]).view(S, KV, DH), pos, f)
        v = F.linear(x, w[p + "mixer.wv.weight"]).view(S, KV, DH)
        rows = []
        for i in range(S):
            lo = max(i - win + 1, 0) if win else 0
            rows.append(plain.attention(q[i : i + 1], k[lo : i + 1], v[lo : i + 1]))
        h = h + F.linear(torch.cat(rows), w[p + "mixer.wo.weight"])
        h = h + plain.swiglu(plain.rms_norm(h, w[p + "ffn_norm.weight"], 1e-5), w[p + "ffn.w1.weight"], w[p + "ffn.w3.weight"], w[p + "ffn.w2.weight"])
    return F.linear(plain.rms_norm(h, w["final_norm.weight"], 1e-5), w["embed.weight"])
