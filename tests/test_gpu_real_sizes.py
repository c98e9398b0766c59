"""The engine at the layer sizes of a real model (hidden 4096, 32 heads in 8 groups of head size
128, feed-forward 14336, llama3 rope scaling; two layers and a small vocabulary to keep it quick):
the kernels' paths that tiny configurations do not reach (the decode products' measured launch
choices, the MFMA attention kernels at head size 128, long rows in the norms)."""

import pytest
import torch

from . import schedules
from .helpers import make_folder, random_tokens, read_folder
from .plain import llama as plain
from .test_gpu_engine import FP32_ATOL, run_trace

pytestmark = pytest.mark.gpu

REAL = dict(
    architectures=["LlamaForCausalLM"], hidden_size=4096, num_hidden_layers=2, num_attention_heads=32,
    num_key_value_heads=8, head_dim=128, intermediate_size=14336, vocab_size=1000, rms_norm_eps=1e-5,
    rope_theta=500000.0, max_position_embeddings=8192, tie_word_embeddings=False,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
)
LENGTHS = [150, 70, 333, 40]


def _bf16_tolerance(weights, cfg, tokens, want):
    yard = plain.forward(weights, cfg, tokens, torch.bfloat16, device="cuda:0").float().cpu()
    return 2 * (yard - want).abs().amax(dim=-1) + 1e-3  # per position


@pytest.fixture(scope="module")
def real(tmp_path_factory):
    folder = make_folder(tmp_path_factory.mktemp("real") / "m", REAL, seed=3, dtype=torch.bfloat16, norm_jitter=0.1, sharpen=True)
    cfg, weights = read_folder(folder)
    requests = {f"r{i}": random_tokens(n, REAL["vocab_size"], 40 + i) for i, n in enumerate(LENGTHS)}
    truth = {rid: plain.forward(weights, cfg, t, torch.float32) for rid, t in requests.items()}
    yard = {rid: plain.forward(weights, cfg, t, torch.bfloat16).float() for rid, t in requests.items()}
    traces = {"whole": schedules.whole(requests), "tail": schedules.tail(requests), "mixed": schedules.mixed(requests)}
    return folder, requests, truth, yard, traces


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_real_layer_sizes_match_the_plain_model_under_every_schedule(real, dtype):
    from torchllms_amd.engine import Engine

    folder, requests, truth, yard, traces = real
    pool_tokens = max(schedules.max_live_tokens(t) for t in traces.values())
    eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=-(-pool_tokens // 16), max_seqs=4)
    results = {name: run_trace(eng, trace) for name, trace in traces.items()}
    for name, res in results.items():
        for (rid, pos), row in res.items():
            want = truth[rid][pos]
            if dtype == "float32":
                err = (row - want).abs().max().item()
                assert err < 10 * FP32_ATOL, f"{name}: {rid} position {pos}: {err}"  # sums are 64 times longer than in the tiny models
            else:
                tol = 2 * (yard[rid][pos] - want).abs().max().item() + 1e-3
                assert (row - want).abs().max().item() <= tol, f"{name}: {rid} position {pos}"
    if dtype == "float32":
        for name in ("tail", "mixed"):
            for key, row in results[name].items():
                assert torch.equal(row, results["whole"][key]), f"{name} differs from whole at {key}"


# the largest shape that is benchmarked: hidden 8192, 64 heads in 8 groups of 8, feed-forward 28672 (Llama-3.1-70B), one layer
LARGE = dict(REAL, num_hidden_layers=1, hidden_size=8192, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
             intermediate_size=28672)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_largest_layer_sizes_match_the_plain_model(tmp_path_factory, dtype):
    """Eight query heads per kv head, rows of 8,192 in the norms (the widest the norm that adds split sums
    takes), matrices of 8,192 x 28,672: whole requests and the mixed schedule, with pages used again."""
    from torchllms_amd.engine import Engine

    folder = make_folder(tmp_path_factory.mktemp("large") / "m", LARGE, seed=9, dtype=torch.bfloat16, norm_jitter=0.1, sharpen=True)
    cfg, weights = read_folder(folder)
    requests = {f"r{i}": random_tokens(n, LARGE["vocab_size"], 60 + i) for i, n in enumerate([150, 70, 333, 40])}
    truth = {rid: plain.forward(weights, cfg, t, torch.float32) for rid, t in requests.items()}
    traces = {"whole": schedules.whole(requests), "mixed": schedules.mixed(requests)}
    pool_tokens = max(schedules.max_live_tokens(t) for t in traces.values())
    eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=-(-pool_tokens // 16), max_seqs=4)
    results = {name: run_trace(eng, trace) for name, trace in traces.items()}
    tols = {rid: _bf16_tolerance(weights, cfg, t, truth[rid]) for rid, t in requests.items()} if dtype == "bfloat16" else None
    for name, res in results.items():
        for (rid, pos), row in res.items():
            err = (row - truth[rid][pos]).abs().max().item()
            if dtype == "float32":
                assert err < 10 * FP32_ATOL, f"{name}: {rid} position {pos}: {err}"
            else:
                assert err <= tols[rid][pos].item(), f"{name}: {rid} position {pos}: {err} against {tols[rid][pos].item()}"
    if dtype == "float32":
        for key, row in results["mixed"].items():
            assert torch.equal(row, results["whole"][key]), f"mixed differs from whole at {key}"


# ----------------------------------------------------------------------------- the sizes that are benchmarked
# One layer of the same sizes: long prompts (a prefill launch of more than 1,024 blocks, portions behind a
# long prefix), decode steps replayed from graphs across context caps, and many live requests of very
# unequal lengths.  The 32-bit truth is the plain model on the CPU; the bfloat16 yardstick is the plain
# model in bfloat16, whose tensor operations torch runs on the GPU here (on the CPU they take minutes).
ONE_LAYER = dict(REAL, num_hidden_layers=1)


@pytest.fixture(scope="module")
def one_layer(tmp_path_factory):
    folder = make_folder(tmp_path_factory.mktemp("long") / "m", ONE_LAYER, seed=5, dtype=torch.bfloat16, norm_jitter=0.1, sharpen=True)
    cfg, weights = read_folder(folder)
    return folder, cfg, weights


def _cut(rid, tokens, sizes, tail):
    """A trace of one request: portions of the given sizes, then ``tail`` single tokens, all wanted."""
    steps, i = [], 0
    for n in list(sizes) + [1] * tail:
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": tokens[i : i + n], "want": list(range(n))}], "end": []})
        i += n
    assert i == len(tokens)
    steps[-1]["end"] = [rid]
    return steps


# the other shape that is benchmarked: hidden 2048, head size 64, tied head, rope factor 32 (Llama-3.2-1B)
ONE_LAYER_SMALL = dict(
    REAL, num_hidden_layers=1, hidden_size=2048, head_dim=64, intermediate_size=8192, tie_word_embeddings=True,
    rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
)


@pytest.fixture(scope="module")
def one_layer_small(tmp_path_factory):
    folder = make_folder(tmp_path_factory.mktemp("small") / "m", ONE_LAYER_SMALL, seed=6, dtype=torch.bfloat16, norm_jitter=0.1, sharpen=True)
    cfg, weights = read_folder(folder)
    return folder, cfg, weights


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_at_head_size_64(one_layer_small, dtype):
    """The same at the 1B shape's sizes: the MFMA attention kernels of head size 64 behind long prefixes, a
    tied head, another rope factor."""
    _long_prompt(one_layer_small, dtype, head_dim=64)


# head size 256, four query heads per kv head: the attention kernels' other tile sizes
ONE_LAYER_WIDE_HEADS = dict(REAL, num_hidden_layers=1, hidden_size=2048, num_attention_heads=8, num_key_value_heads=2, head_dim=256,
                            intermediate_size=4096)


@pytest.fixture(scope="module")
def one_layer_wide_heads(tmp_path_factory):
    folder = make_folder(tmp_path_factory.mktemp("wide") / "m", ONE_LAYER_WIDE_HEADS, seed=7, dtype=torch.bfloat16, norm_jitter=0.1, sharpen=True)
    cfg, weights = read_folder(folder)
    return folder, cfg, weights


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_at_head_size_256(one_layer_wide_heads, dtype):
    _long_prompt(one_layer_wide_heads, dtype, head_dim=256, heads=8, kv_heads=2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_whole_and_in_portions_behind_a_long_prefix(one_layer, dtype):
    """4,700 tokens in one step (1,176 blocks of the prefill attention kernel: beyond the 1,024 up
    to which blocks hold two sets of waves), then the same request as 2,100 tokens, portions of 700,
    2, 1,000, 31 and 827 behind them, and the last 40 tokens one by one."""
    _long_prompt(one_layer, dtype, head_dim=128)


def _long_prompt(model, dtype, head_dim, heads=32, kv_heads=8, one_set_of_waves=True):
    from torchllms_amd.engine import Engine
    from torchllms_amd.kernels import ops

    folder, cfg, weights = model
    n = 4700
    tokens = random_tokens(n, ONE_LAYER["vocab_size"], 77)
    want = plain.forward(weights, cfg, tokens, torch.float32)
    qpt = ops.prefill_queries_per_tile(heads, kv_heads, head_dim)
    # the whole prompt is a launch with one set of waves a block, or with two
    assert (ops.prefill_key_groups(-(-n // qpt), kv_heads, n) == 1) == one_set_of_waves
    eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=-(-n // 16) + 1, max_seqs=2, max_model_len=8192)
    whole = run_trace(eng, _cut("w", tokens, [n], 0))
    parts = run_trace(eng, _cut("p", tokens, [2100, 700, 2, 1000, 31, 827], 40))
    tol = _bf16_tolerance(weights, cfg, tokens, want) if dtype == "bfloat16" else None
    for name, res in (("whole", whole), ("portions", parts)):
        rid = name[0]
        got = torch.stack([res[(rid, pos)] for pos in range(n)])
        err = (got - want).abs().amax(dim=-1)
        if dtype == "float32":
            bad = (err >= 10 * FP32_ATOL).nonzero().flatten()
        else:
            bad = (err > tol).nonzero().flatten()
        assert bad.numel() == 0, f"{name}: first wrong position {int(bad[0])} of {bad.numel()}, error {err[bad[0]].item()}"
    if dtype == "float32":
        diff = [pos for pos in range(n) if not torch.equal(whole[("w", pos)], parts[("p", pos)])]
        assert not diff, f"portions differ from the whole prompt at {len(diff)} positions, first {diff[0]}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_graphs_across_context_caps(one_layer, dtype):
    """Two requests decoded side by side from 480 and 30 tokens on, one token a step, until the
    longer holds 2,070: the recorded decode steps change with the context cap (512, 768, 1,024, ...
    3,072), each with wider block tables and more splits of the keys."""
    from torchllms_amd.engine import Engine

    folder, cfg, weights = one_layer
    long_tokens = random_tokens(2070, ONE_LAYER["vocab_size"], 78)
    short_tokens = random_tokens(30 + 1590, ONE_LAYER["vocab_size"], 79)
    want = {"a": plain.forward(weights, cfg, long_tokens, torch.float32), "b": plain.forward(weights, cfg, short_tokens, torch.float32)}
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": long_tokens[:480], "want": list(range(480))},
                                     {"id": "b", "tokens": short_tokens[:30], "want": list(range(30))}], "end": []}]
    for i in range(1590):
        steps.append({"step": len(steps), "entries": [{"id": "a", "tokens": [long_tokens[480 + i]], "want": [0]},
                                                      {"id": "b", "tokens": [short_tokens[30 + i]], "want": [0]}], "end": []})
    steps[-1]["end"] = ["a", "b"]
    eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=2 * 130 + 2, max_seqs=2, max_model_len=4096, use_graphs=True)
    got = run_trace(eng, steps)
    caps = sorted(key[2] for key in eng.graphs.graphs)
    assert set(caps) == {512, 768, 1024, 1536, 2048, 3072}, caps
    assert sum(g.replays for g in eng.graphs.graphs.values()) > 1500
    tols = {r: _bf16_tolerance(weights, cfg, t, want[r]) for r, t in (("a", long_tokens), ("b", short_tokens))} if dtype == "bfloat16" else None
    for rid, toks in (("a", long_tokens), ("b", short_tokens)):
        rows = torch.stack([got[(rid, pos)] for pos in range(len(toks))])
        err = (rows - want[rid]).abs().amax(dim=-1)
        bad = (err >= 10 * FP32_ATOL).nonzero().flatten() if dtype == "float32" else (err > tols[rid]).nonzero().flatten()
        assert bad.numel() == 0, f"{rid}: first wrong position {int(bad[0])} of {bad.numel()}, error {err[bad[0]].item()}"
    if dtype == "float32":
        # the same bits as the whole prompt in one step gives
        whole = run_trace(eng, _cut("a", long_tokens, [len(long_tokens)], 0))
        diff = [pos for pos in range(len(long_tokens)) if not torch.equal(whole[("a", pos)], got[("a", pos)])]
        assert not diff, f"decoded positions differ from the whole prompt at {len(diff)} positions, first {diff[0]}"


MANY_LENGTHS = [1900, 23, 700, 64, 1100, 17, 1500] + [10 + (37 * i) % 111 for i in range(57)]  # 64 requests, very unequal


@pytest.fixture(scope="module")
def many(one_layer):
    folder, cfg, weights = one_layer
    requests = {f"m{i}": random_tokens(n, ONE_LAYER["vocab_size"], 300 + i) for i, n in enumerate(MANY_LENGTHS)}
    truth = {rid: plain.forward(weights, cfg, t, torch.float32) for rid, t in requests.items()}
    return requests, truth


@pytest.mark.parametrize("live", [24, 64])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_many_live_requests_of_unequal_lengths_decode_together(one_layer, many, dtype, live):
    """24 and 64 live requests of 10 to 1,900 tokens: prompts prefilled eight to a step, then the
    last 20 tokens of every request decoded together, 24 or 64 rows a step, replayed from graphs
    whose key says that the lengths differ much (shorter key splits in the decode attention)."""
    _many_live(one_layer, many, dtype, live)


@pytest.fixture(scope="module")
def many_small(one_layer_small):
    folder, cfg, weights = one_layer_small
    requests = {f"m{i}": random_tokens(n, ONE_LAYER["vocab_size"], 300 + i) for i, n in enumerate(MANY_LENGTHS)}
    truth = {rid: plain.forward(weights, cfg, t, torch.float32) for rid, t in requests.items()}
    return requests, truth


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_many_live_requests_at_head_size_64(one_layer_small, many_small, dtype):
    """The same with 64 live requests at the 1B shape's sizes: the decode attention of head size 64 and the
    decode products of a hidden size of 2,048, replayed from graphs."""
    _many_live(one_layer_small, many_small, dtype, 64)


def _many_live(model, many, dtype, live):
    from torchllms_amd.engine import Engine

    folder, cfg, weights = model
    all_requests, truth = many
    requests = dict(list(all_requests.items())[:live])
    tail = 20
    steps = []
    rids = list(requests)
    for lo in range(0, live, 8):
        group = rids[lo : lo + 8]
        steps.append({"step": len(steps), "end": [], "entries": [
            {"id": r, "tokens": requests[r][: len(requests[r]) - tail], "want": [len(requests[r]) - tail - 1]} for r in group if len(requests[r]) > tail]})
    for i in range(tail):
        entries = []
        for r in rids:
            n = len(requests[r])
            if n > tail:
                entries.append({"id": r, "tokens": [requests[r][n - tail + i]], "want": [0]})
            elif i == 0:
                entries.append({"id": r, "tokens": requests[r], "want": [n - 1]})  # a short prompt joins whole
        steps.append({"step": len(steps), "entries": entries, "end": []})
    steps[-1]["end"] = rids
    pages = sum(-(-len(t) // 16) for t in requests.values()) + 4
    eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=pages, max_seqs=live, max_model_len=4096, use_graphs=True)
    got = run_trace(eng, steps)
    n_rows = sum(1 for r in rids if len(requests[r]) > tail)
    assert any(key[0] == n_rows and key[3] for key in eng.graphs.graphs), list(eng.graphs.graphs)  # rows, uneven lengths
    assert sum(g.replays for g in eng.graphs.graphs.values()) >= tail - 4
    worst = []
    for (rid, pos), row in got.items():
        want = truth[rid][pos]
        err = (row - want).abs().max().item()
        if dtype == "float32":
            assert err < 10 * FP32_ATOL, f"{rid} position {pos}: {err}"
        else:
            worst.append((err, rid, pos))
    if dtype == "bfloat16":
        tols = {r: _bf16_tolerance(weights, cfg, requests[r], truth[r]) for r in {rid for _, rid, _ in worst}}
        for err, rid, pos in worst:
            assert err <= tols[rid][pos].item(), f"{rid} position {pos}: {err} against {tols[rid][pos].item()}"


# ----------------------------------------------------------------------------- context 8,192: the sizes of the headline measurement
def _plain_on_gpu(weights, cfg, tokens, dtype):
    """The plain model's logits with torch's tensor operations run on the GPU (the same functions; a
    sequence of 8,192 tokens takes minutes on the CPU), back on the CPU as 32-bit."""
    out = plain.forward(weights, cfg, tokens, dtype, device="cuda:0").float().cpu()
    torch.cuda.empty_cache()
    return out


def _check_rows(name, got, want, dtype, tol):
    err = (got - want).abs().amax(dim=-1)
    bad = (err >= 10 * FP32_ATOL).nonzero().flatten() if dtype == "float32" else (err > tol).nonzero().flatten()
    assert bad.numel() == 0, f"{name}: first wrong position {int(bad[0])} of {bad.numel()}, error {err[bad[0]].item()}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_request_of_8192_tokens_whole_in_portions_and_decoded_across_the_last_context_caps(one_layer, dtype):
    """One request that fills the context of 8,192: in one step (a prefill launch of 2,048 blocks); in
    portions of 4,096, 2, 3,000, 31 and 971 tokens with the last 92 one by one; and with three runs of
    decode steps, at contexts 4,061 to 4,120, 6,121 to 6,180 and 8,101 to 8,192, replayed from graphs
    recorded for the context caps 4,096, 6,144 and 8,192 (the widest block tables and the most key
    splits of the decode attention), prompt portions of about 2,000 tokens in between."""
    from torchllms_amd.engine import Engine

    folder, cfg, weights = one_layer
    n = 8192
    tokens = random_tokens(n, ONE_LAYER["vocab_size"], 81)
    want = _plain_on_gpu(weights, cfg, tokens, torch.float32)
    tol = 2 * (_plain_on_gpu(weights, cfg, tokens, torch.bfloat16) - want).abs().amax(dim=-1) + 1e-3 if dtype == "bfloat16" else None
    eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=n // 16 + 1, max_seqs=2, max_model_len=n, use_graphs=True)
    results = {"whole": run_trace(eng, _cut("w", tokens, [n], 0))}
    assert not eng.graphs.graphs
    results["portions"] = run_trace(eng, _cut("p", tokens, [4096, 2, 3000, 31, 971], 92))
    caps = sorted(key[2] for key in eng.graphs.graphs)
    assert caps == [8192], caps
    sizes = [4060] + [1] * 60 + [2000] + [1] * 60 + [1920]
    results["decoded"] = run_trace(eng, _cut("d", tokens, sizes, 92))
    caps = sorted(key[2] for key in eng.graphs.graphs)
    assert caps == [4096, 6144, 8192], caps
    assert sum(g.replays for g in eng.graphs.graphs.values()) >= 92 + 212 - 4 * 3
    rows = {name: torch.stack([res[(name[0], pos)] for pos in range(n)]) for name, res in results.items()}
    for name, got in rows.items():
        _check_rows(name, got, want, dtype, tol)
    if dtype == "float32":
        for name in ("portions", "decoded"):
            diff = (rows[name] != rows["whole"]).any(dim=-1).nonzero().flatten()
            assert diff.numel() == 0, f"{name} differs from the whole prompt at {diff.numel()} positions, first {int(diff[0])}"


class _Recorder:
    """An engine as the generation loop sees it, which keeps the logits of every step by (request,
    position).  Every way in which the loop runs a step goes through here."""

    def __init__(self, engine):
        self.engine, self.cache, self.rows = engine, engine.cache, {}
        self.ways = {"step": 0, "step_prepared": 0, "step_prepared_on_device": 0}

    def _note(self, way, wanted, logits):
        if logits is None:
            return None
        self.ways[way] += 1
        places = [(rid, self.cache.num_tokens(rid) - n + w) for rid, n, want in wanted for w in want]
        assert logits.shape[0] == len(places)
        for place, row in zip(places, logits.clone()):
            assert place not in self.rows
            self.rows[place] = row
        return logits

    def step(self, entries):
        return self._note("step", [(e.rid, len(e.tokens), e.want) for e in entries], self.engine.step(entries))

    def prepare_decode(self):
        return self.engine.prepare_decode()

    def step_prepared(self, prepared, entries):
        return self._note("step_prepared", [(e.rid, 1, e.want) for e in entries], self.engine.step_prepared(prepared, entries))

    def step_prepared_on_device(self, prepared, rids, token_ids):
        return self._note("step_prepared_on_device", [(rid, 1, [0]) for rid in rids],
                          self.engine.step_prepared_on_device(prepared, rids, token_ids))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_eight_requests_at_context_8192_through_the_generation_loop(one_layer, dtype):
    """The shape whose speed is the headline figure: eight requests with prompts of 8,152 tokens,
    admitted and cut into portions by the scheduler under a token budget of 8,192 (the first decodes
    while the others' prompts come in), then 40 tokens generated for each, the decode steps of all eight
    replayed from one graph at the context cap 8,192 and launched ahead of the host.  The logits of
    every sampled position against the plain model run over the prompt and what was generated."""
    from torchllms_amd.engine import Engine
    from torchllms_amd.inference.llm import GenerationLoop
    from torchllms_amd.sampling import Sampler, SamplingParams

    folder, cfg, weights = one_layer
    batch, prompt_len, new = 8, 8152, 40
    prompts = [random_tokens(prompt_len, ONE_LAYER["vocab_size"], 500 + i) for i in range(batch)]
    eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=batch * 513, max_seqs=batch, max_model_len=8192, use_graphs=True)
    rec = _Recorder(eng)
    loop = GenerationLoop(rec, Sampler(), max_num_seqs=batch, max_num_batched_tokens=8192, max_model_len=8192)
    params = [SamplingParams(temperature=0.0, max_new_tokens=new, stop_token_ids=(), seed=i) for i in range(batch)]
    requests = loop.run(prompts, params)
    assert all(len(r.output) == new for r in requests)
    eng.cache.check_invariants()
    graph = eng.graphs.graphs.get((batch, batch, 8192, False))
    assert graph is not None and graph.replays >= 20, {k: g.replays for k, g in eng.graphs.graphs.items()}
    assert rec.ways["step_prepared_on_device"] >= 15, rec.ways
    assert len(rec.rows) == batch * new
    for i, r in enumerate(requests):
        tokens = prompts[i] + list(r.output)
        want = _plain_on_gpu(weights, cfg, tokens, torch.float32)
        tol = 2 * (_plain_on_gpu(weights, cfg, tokens, torch.bfloat16) - want).abs().amax(dim=-1) + 1e-3 if dtype == "bfloat16" else None
        places = [pos for (rid, pos) in rec.rows if rid == r.rid]
        assert sorted(places) == list(range(prompt_len - 1, prompt_len + new - 1)), (i, sorted(places)[:3])
        got = torch.stack([rec.rows[(r.rid, pos)].cpu() for pos in sorted(places)])
        _check_rows(f"request {i}", got, want[prompt_len - 1 : prompt_len + new - 1], dtype, None if tol is None else tol[prompt_len - 1 : prompt_len + new - 1])
        # greedy: each generated token is the plain model's choice wherever that choice is clear
        top2 = want[prompt_len - 1 : prompt_len + new - 1].topk(2, dim=-1)
        margin = 20 * FP32_ATOL if dtype == "float32" else 2 * tol[prompt_len - 1 : prompt_len + new - 1]
        clear = (top2.values[:, 0] - top2.values[:, 1]) > margin
        assert clear.any()
        assert torch.equal(torch.tensor(r.output)[clear], top2.indices[:, 0][clear]), f"request {i}"
