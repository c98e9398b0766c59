"""Generation through the Python entry point and the command line, on the GPU."""

import json
import subprocess
import sys
from pathlib import Path

import pytest
import torch

from .helpers import TINY, make_folder, random_tokens, read_folder
from .plain import llama as plain

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    folder = make_folder(tmp_path_factory.mktemp("gen") / "B", TINY["B"], seed=5, dtype=torch.bfloat16, sharpen=True)
    cfg, weights = read_folder(folder)
    return folder, cfg, weights


def plain_greedy(weights, cfg, prompt, n, stop=()):
    toks = list(prompt)
    for _ in range(n):
        nxt = int(plain.forward(weights, cfg, toks, torch.float32)[-1].argmax())
        toks.append(nxt)
        if nxt in stop:
            break
    return toks[len(prompt):]


def test_greedy_generation_matches_the_plain_model(model_b):
    from torchllms_amd.inference import LLM

    folder, cfg, weights = model_b
    prompts = [random_tokens(n, cfg["vocab_size"], 40 + n) for n in (5, 17, 1, 32)]
    llm = LLM(str(folder), precision="float32", max_len=128, max_bsz=3, page_size=8)
    results = llm.generate(prompt_token_ids=prompts, temperature=0.0, max_new_tokens=12)
    for p, r in zip(prompts, results):
        assert r.token_ids == plain_greedy(weights, cfg, p, 12) and r.stop_reason is None and r.text == ""
    # a stop token ends the request and is kept
    want = plain_greedy(weights, cfg, prompts[1], 12)
    stop = want[4]
    r = llm.generate(prompt_token_ids=[prompts[1]], max_new_tokens=12, stop_token_ids=[stop])[0]
    cut = want.index(stop) + 1
    assert r.token_ids == want[:cut] and r.stop_reason == stop
    llm.engine.cache.check_invariants()
    assert llm.engine.cache.live == []


def test_bfloat16_greedy_picks_tokens_the_plain_model_rates_highest(model_b):
    from torchllms_amd.inference import LLM

    folder, cfg, weights = model_b
    prompt = random_tokens(20, cfg["vocab_size"], 77)
    llm = LLM(str(folder), precision="bfloat16", max_len=128, max_bsz=2)
    got = llm.generate(prompt_token_ids=[prompt], max_new_tokens=16)[0].token_ids
    assert len(got) == 16
    toks = prompt + got
    logits32 = plain.forward(weights, cfg, toks, torch.float32)
    logits16 = plain.forward(weights, cfg, toks, torch.bfloat16).float()
    slack = 2 * (logits16 - logits32).abs().max().item()
    for i, tok in enumerate(got):
        row = logits32[len(prompt) - 1 + i]
        assert row[tok] >= row.max() - slack, f"token {i}: chose {tok}, plain model prefers {int(row.argmax())}"


def test_seeded_sampling_does_not_depend_on_batch_mates(model_b):
    from torchllms_amd.inference import LLM

    folder, cfg, _ = model_b
    prompts = [random_tokens(n, cfg["vocab_size"], 60 + n) for n in (1, 9, 40, 100)]
    llm = LLM(str(folder), precision="float32", max_len=160, max_bsz=4, max_num_batched_tokens=24)
    together = llm.generate(prompt_token_ids=prompts, temperature=0.7, max_new_tokens=24, seed=1234)
    assert llm.last_stats["steps"] > 24  # prompts were fed in 24-token portions beside decoding
    for i, p in enumerate(prompts):
        alone = llm.generate(prompt_token_ids=[p], temperature=0.7, max_new_tokens=24, seed=1234 + i)[0]
        assert alone.token_ids == together[i].token_ids
    other = llm.generate(prompt_token_ids=prompts, temperature=0.7, max_new_tokens=24, seed=99)
    assert [r.token_ids for r in other] != [r.token_ids for r in together]
    greedy = llm.generate(prompt_token_ids=prompts, temperature=0.0, max_new_tokens=24)
    assert [r.token_ids for r in greedy] != [r.token_ids for r in together]


def test_preemption_on_the_gpu_changes_nothing(model_b):
    from torchllms_amd.inference import LLM

    folder, cfg, _ = model_b
    prompts = [random_tokens(n, cfg["vocab_size"], 80 + n) for n in (30, 25, 28, 21)]
    ample = LLM(str(folder), precision="float32", max_len=96, max_bsz=4, page_size=8)
    want = ample.generate(prompt_token_ids=prompts, temperature=0.8, max_new_tokens=30, seed=7)
    tight = LLM(str(folder), precision="float32", max_len=96, max_bsz=4, page_size=8, num_pages=20)  # 160 places for 224 tokens
    got = tight.generate(prompt_token_ids=prompts, temperature=0.8, max_new_tokens=30, seed=7)
    assert tight.last_stats["preemptions"] > 0
    assert [r.token_ids for r in got] == [r.token_ids for r in want]
    tight.engine.cache.check_invariants()


@pytest.mark.parametrize("precision", ["float32", "bfloat16"])
def test_preparing_the_next_step_ahead_changes_no_token(model_b, precision):
    """Seven requests of different lengths and budgets, three at a time, some ending on a stop
    token: with the next decode step prepared during the current one, the tokens are those of the
    loop that plans every step when it runs, and most decode steps did run prepared."""
    from torchllms_amd.inference import LLM

    folder, cfg, _ = model_b
    prompts = [random_tokens(n, cfg["vocab_size"], 300 + n) for n in (3, 50, 17, 8, 33, 1, 25)]
    llm = LLM(str(folder), precision=precision, max_len=160, max_bsz=3, page_size=8, max_num_batched_tokens=32)
    assert llm.engine.graphs is not None
    llm.look_ahead = False
    base = llm.generate(prompt_token_ids=prompts, temperature=0.9, max_new_tokens=60, seed=5)
    assert llm.last_stats["prepared_steps"] == 0
    stops = [base[1].token_ids[20], base[4].token_ids[41]]  # end two of them early
    want = llm.generate(prompt_token_ids=prompts, temperature=0.9, max_new_tokens=60, seed=5, stop_token_ids=stops)
    steps = llm.last_stats["steps"]
    assert any(r.stop_reason is not None for r in want) and any(r.stop_reason is None for r in want)
    llm.look_ahead = True
    # a step launched ahead has its tokens written by the sampling kernel where it reads them: no copy, and the plan
    # goes up without them
    from torchllms_amd.engine.graphs import DecodeGraph

    in_place = []
    upload = DecodeGraph._upload

    def counting(self, but_tokens=0):
        in_place.append(but_tokens)
        return upload(self, but_tokens)

    DecodeGraph._upload = counting
    try:
        got = llm.generate(prompt_token_ids=prompts, temperature=0.9, max_new_tokens=60, seed=5, stop_token_ids=stops)
    finally:
        DecodeGraph._upload = upload
    assert [r.token_ids for r in got] == [r.token_ids for r in want]
    assert [r.stop_reason for r in got] == [r.stop_reason for r in want]
    assert llm.last_stats["steps"] == steps and llm.last_stats["prepared_steps"] > steps // 3
    assert llm.last_stats["launched_ahead"] > steps // 4  # queued behind the sampling, before the host had the tokens
    assert sum(1 for n in in_place if n > 0) == llm.last_stats["launched_ahead"]
    llm.engine.cache.check_invariants()
    assert llm.engine.cache.live == []


@pytest.mark.parametrize("precision", ["float32", "bfloat16"])
def test_steps_launched_ahead_cope_with_requests_that_end(model_b, precision):
    """A decode step that is launched with the sampled tokens still on the device is wrong for a
    request that ends on that very token.  Many requests with a fifth of the vocabulary as stop
    tokens, four at a time with others waiting, greedy and sampled, with ample pages; and with a
    twenty-third of it and so few pages that running requests are preempted for want of pages, in
    the loop that launches ahead as in the other: the tokens and stop reasons are those of the loop
    that waits for the tokens before every step, and every page comes back."""
    from torchllms_amd.inference import LLM

    folder, cfg, _ = model_b
    vocab = cfg["vocab_size"]
    prompts = [random_tokens(3 + (11 * i) % 40, vocab, 500 + i) for i in range(14)]
    for pages, temperature in ((None, 0.0), (None, 1.3), (16, 1.3)):
        kw = dict(num_pages=pages) if pages else {}
        stops = list(range(0, vocab, 23 if pages else 5))
        llm = LLM(str(folder), precision=precision, max_len=120, max_bsz=4, page_size=8, max_num_batched_tokens=24, **kw)
        llm.look_ahead = False
        want = llm.generate(prompt_token_ids=prompts, temperature=temperature, max_new_tokens=40, seed=11, stop_token_ids=stops)
        assert sum(r.stop_reason is not None for r in want) >= 5 and llm.last_stats["launched_ahead"] == 0
        assert not pages or llm.last_stats["preemptions"] > 0
        llm.look_ahead = True
        got = llm.generate(prompt_token_ids=prompts, temperature=temperature, max_new_tokens=40, seed=11, stop_token_ids=stops)
        assert [r.token_ids for r in got] == [r.token_ids for r in want], (pages, temperature)
        assert [r.stop_reason for r in got] == [r.stop_reason for r in want]
        assert llm.last_stats["launched_ahead"] > 0
        assert not pages or llm.last_stats["preemptions"] > 0
        llm.engine.cache.check_invariants()
        assert llm.engine.cache.live == [] and llm.engine.cache.free_pages() == llm.engine.cache.pools[0].num_pages


def test_generate_command_line(model_b, tmp_path):
    folder, cfg, weights = model_b
    prompts = [random_tokens(n, cfg["vocab_size"], 90 + n) for n in (4, 11)]
    inp, out = tmp_path / "in.jsonl", tmp_path / "sub" / "out.jsonl"
    inp.write_text("".join(json.dumps({"prompt_token_ids": p, "tag": i}) + "\n" for i, p in enumerate(prompts)))
    cmd = [
        sys.executable, "-m", "torchllms_amd.inference.generate", "--input_path", str(inp), "--output_path", str(out),
        "--provider_kwargs", json.dumps({"ckpt_paths": str(folder), "precision": "float32", "max_len": 64}),
        "--generate_kwargs", json.dumps({"max_new_tokens": 5}),
    ]
    subprocess.run(cmd, check=True, cwd=ROOT, timeout=300)
    recs = [json.loads(l) for l in out.read_text().splitlines()]
    assert [r["tag"] for r in recs] == [0, 1]
    for p, r in zip(prompts, recs):
        assert r["completion_token_ids"] == plain_greedy(weights, cfg, p, 5)


def test_smoke_entry():
    sys.path.insert(0, str(ROOT))
    import __graft_entry__

    __graft_entry__.smoke()
