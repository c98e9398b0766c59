"""The scheduler's decisions and the generation loop, on the CPU with a fake engine.

The fake engine keeps the real cache manager's books and answers, for a token at position p, with
logits whose argmax is (p + 1) % VOCAB, as the reference's own fake model does.  Vectors marked
(ref) restate reference: torchllms/inference/test_prefix_cache_wiring.py:257-555.
"""

import random

import pytest
import torch

from torchllms_amd.cache import CacheGroupSpec, CacheManager
from torchllms_amd.engine.scheduler import Scheduler
from torchllms_amd.inference.llm import GenerationLoop
from torchllms_amd.sampling import SamplingParams

VOCAB = 32


class FakeEngine:
    def __init__(self, num_pages=64, page_size=4, max_seqs=4, window=0, groups=None):
        groups = groups or [CacheGroupSpec("kv0", (0,), 1, 4, window)]
        self.cache = CacheManager(groups, [], page_size, num_pages, max_seqs)
        self.calls = []  # per step: list of (rid, first position, n tokens)

    def step(self, entries):
        need = [sum(per_group) for per_group in zip(*(self.cache.new_pages_needed(e.rid, len(e.tokens)) for e in entries))]
        for g, n in enumerate(need):
            assert n <= self.cache.free_pages(g), "the scheduler planned a step the pool cannot hold"
        rows, call = [], []
        for e in entries:
            start = self.cache.extend(e.rid, len(e.tokens))
            call.append((e.rid, start, len(e.tokens)))
            for w in e.want:
                row = torch.zeros(VOCAB)
                row[(start + w + 1) % VOCAB] = 1.0
                rows.append(row)
        for e in entries:
            self.cache.advance(e.rid, len(e.tokens))
        self.cache.check_invariants()
        self.calls.append(call)
        return torch.stack(rows) if rows else torch.zeros(0, VOCAB)


def greedy(logits, params, steps):
    return logits.argmax(-1).tolist() if len(params) else []


def generate(prompts, max_new_tokens=None, stop=(), engine=None, max_num_seqs=4, budget=64, max_model_len=256, chunk=None):
    engine = engine or FakeEngine()
    loop = GenerationLoop(engine, greedy, max_num_seqs, budget, max_model_len, chunk)
    params = [SamplingParams(max_new_tokens=max_new_tokens, stop_token_ids=stop) for _ in prompts]
    reqs = loop.run(prompts, params)
    assert engine.cache.live == [] and all(engine.cache.free_pages(g) == p.num_pages for g, p in enumerate(engine.cache.pools))
    return reqs, engine, loop


def test_single_request_token_stream_and_call_count():  # (ref)
    reqs, eng, _ = generate([[5, 6, 7, 8, 9]], max_new_tokens=6)
    assert reqs[0].output == [5, 6, 7, 8, 9, 10] and reqs[0].stop_reason is None
    assert len(eng.calls) == 6 and eng.calls[0][0][2] == 5 and all(c[0][2] == 1 for c in eng.calls[1:])


def test_zero_budget_runs_nothing():  # (ref)
    reqs, eng, _ = generate([[5, 6, 7]], max_new_tokens=0)
    assert reqs[0].output == [] and reqs[0].stop_reason is None and eng.calls == []


def test_stop_ids_are_alternatives_and_the_stop_token_is_kept():  # (ref)
    reqs, _, _ = generate([[5, 6, 7, 8, 9]], max_new_tokens=10, stop=(7, 6))
    assert reqs[0].output == [5, 6] and reqs[0].stop_reason == 6
    reqs, eng, _ = generate([[5, 6, 7, 8, 9]], max_new_tokens=10, stop=(5,))
    assert reqs[0].output == [5] and reqs[0].stop_reason == 5 and len(eng.calls) == 1
    reqs, _, _ = generate([[5, 6, 7, 8, 9]], max_new_tokens=4, stop=(99,))
    assert reqs[0].stop_reason is None and len(reqs[0].output) == 4
    reqs, _, _ = generate([[5, 6, 7, 8, 9]], max_new_tokens=10, stop=(8, 6))
    assert reqs[0].output == [5, 6] and reqs[0].stop_reason == 6


def test_batched_equals_single_per_row_and_order_is_kept():  # (ref: lengths 3, 6, 2)
    prompts = [[1, 2, 3], [1, 2, 3, 4, 5, 6], [7, 8]]
    together, _, _ = generate(prompts, max_new_tokens=5)
    for p, r in zip(prompts, together):
        alone, _, _ = generate([p], max_new_tokens=5)
        assert r.output == alone[0].output == [(len(p) + i) % VOCAB for i in range(5)]
    # rows that finish at different times, one with no budget at all
    loop_reqs, _, _ = generate(prompts, max_new_tokens=None, max_model_len=7)
    assert [len(r.output) for r in loop_reqs] == [4, 1, 5]


def test_context_length_bounds_the_budget():
    reqs, _, _ = generate([[1] * 10], max_new_tokens=100, max_model_len=13)
    assert len(reqs[0].output) == 3
    reqs, eng, _ = generate([[1] * 13], max_new_tokens=100, max_model_len=13)
    assert reqs[0].output == [] and eng.calls == []


def test_empty_prompt_and_impossible_requests_are_refused():
    eng = FakeEngine(num_pages=4, page_size=4)
    s = Scheduler(eng.cache, 4, 64, 256)
    with pytest.raises(ValueError, match="empty prompt"):
        s.add("a", [], SamplingParams(max_new_tokens=3))
    with pytest.raises(ValueError, match="could never finish"):
        s.add("b", [1] * 10, SamplingParams(max_new_tokens=8))  # 17 tokens in the cache > 16 places
    s.add("c", [1] * 10, SamplingParams(max_new_tokens=7))  # 16 tokens: fits exactly


def test_token_budget_and_order_inside_a_step():
    eng = FakeEngine(num_pages=64, page_size=4, max_seqs=4)
    loop = GenerationLoop(eng, greedy, 4, 8, 256)
    seen = []
    prompts = [[1] * 3, [1] * 19, [1] * 6, [1] * 2]
    loop.run(prompts, [SamplingParams(max_new_tokens=6) for _ in prompts], on_step=lambda plan: seen.append(plan))
    assert all(p.n_tokens <= 8 for p in seen)
    # the 19-token prompt was cut into portions; a portion may be as small as the budget leaves
    portions = [n for call in eng.calls for rid, start, n in call if rid[2] == 1 and start < 19]
    assert sum(portions) == 19 and max(portions) <= 8 and len(portions) >= 3
    for p in seen:
        kinds = [len(e.tokens) == 1 and e.samples and len(e.request.output) > 0 for e in p.entries]
        # decoding requests come first, then portions of prompts
        assert kinds == sorted(kinds, reverse=True)
    mixed = [p for p in seen if any(len(e.tokens) > 1 for e in p.entries) and any(len(e.tokens) == 1 for e in p.entries)]
    assert mixed, "no step held a portion of a prompt beside a decoded token"


def test_prefill_chunk_limits_a_portion():
    reqs, eng, _ = generate([[1] * 23], max_new_tokens=2, budget=64, chunk=5)
    sizes = [c[0][2] for c in eng.calls]
    assert sizes == [5, 5, 5, 5, 3, 1]
    assert reqs[0].output == [23, 24]


def test_requests_queue_for_slots():
    prompts = [[1] * (2 + i) for i in range(9)]
    reqs, eng, loop = generate(prompts, max_new_tokens=4, max_num_seqs=2)
    assert all(len(c) <= 2 for c in eng.calls)
    assert [r.output for r in reqs] == [[(2 + i + k) % VOCAB for k in range(4)] for i in range(9)]
    assert loop.scheduler.stats["finished"] == 9


def test_preemption_gives_the_same_tokens_as_an_ample_pool():
    prompts = [[1] * 9, [1] * 7, [1] * 11, [1] * 5]
    ample, _, _ = generate(prompts, max_new_tokens=14)
    tight_engine = FakeEngine(num_pages=12, page_size=4, max_seqs=4)  # 48 places for 32 + 4 * 13 tokens
    tight, _, loop = generate(prompts, max_new_tokens=14, engine=tight_engine)
    assert loop.scheduler.stats["preemptions"] > 0
    assert [r.output for r in tight] == [r.output for r in ample]
    assert any(r.preemptions for r in tight)
    # the oldest request is never the victim
    assert tight[0].preemptions == 0


def test_a_lone_request_that_outgrows_the_pool_is_caught_at_add():
    eng = FakeEngine(num_pages=3, page_size=4)
    loop = GenerationLoop(eng, greedy, 4, 64, 256)
    with pytest.raises(ValueError, match="could never finish"):
        loop.run([[1] * 8], [SamplingParams(max_new_tokens=10)])
    assert eng.cache.live == []


def test_a_window_bounds_what_a_request_must_hold():
    # every group has a window of 6 keys: a request holds the pages those keys touch and no more, so a
    # pool of five pages takes a request of 60 tokens (fifteen pages if none came back), cut into the
    # portions the free pages hold, and generates what an ample pool generates
    prompt = list(range(1, 41))
    tight_engine = FakeEngine(num_pages=5, page_size=4, window=6)
    (tight,), _, _ = generate([prompt], max_new_tokens=20, engine=tight_engine)
    (ample,), _, _ = generate([prompt], max_new_tokens=20, engine=FakeEngine(num_pages=64, page_size=4, window=6))
    assert tight.output == ample.output and len(tight.output) == 20 and tight.preemptions == 0
    assert max(n for call in tight_engine.calls for _, _, n in call) <= 20  # no portion beyond the pool
    # beside a group that keeps every key the request is still refused: that group needs all fifteen
    groups = [CacheGroupSpec("full", ("a",), 1, 4, 0), CacheGroupSpec("windowed", ("b",), 1, 4, 6)]
    loop = GenerationLoop(FakeEngine(num_pages=5, page_size=4, groups=groups), greedy, 4, 64, 256)
    with pytest.raises(ValueError, match="60 tokens need 15 pages"):
        loop.run([prompt], [SamplingParams(max_new_tokens=21)])
    # and a window wider than the pool is refused too
    with pytest.raises(ValueError, match="could never finish"):
        GenerationLoop(FakeEngine(num_pages=2, page_size=4, window=9), greedy, 4, 64, 256).run([prompt], [SamplingParams(max_new_tokens=4)])


def test_failure_gives_everything_back():
    eng = FakeEngine()

    def broken(logits, params, steps):
        if len(eng.calls) >= 3:
            raise RuntimeError("sampler died")
        return greedy(logits, params, steps)

    loop = GenerationLoop(eng, broken, 4, 64, 256)
    with pytest.raises(RuntimeError, match="sampler died"):
        loop.run([[1, 2, 3], [4, 5]], [SamplingParams(max_new_tokens=9)] * 2)
    assert eng.cache.live == [] and eng.cache.free_pages() == 64
    eng.cache.check_invariants()


@pytest.mark.parametrize("seed", range(5))
def test_random_workloads_finish_with_right_tokens(seed):
    rng = random.Random(seed)
    n = rng.randint(3, 12)
    prompts = [[1] * rng.randint(1, 30) for _ in range(n)]
    news = [rng.randint(1, 20) for _ in range(n)]
    page = rng.choice([2, 4, 8])
    longest = max(len(p) + m for p, m in zip(prompts, news))
    eng = FakeEngine(num_pages=-(-longest // page) + rng.randint(0, 6), page_size=page, max_seqs=rng.randint(1, 4))
    loop = GenerationLoop(eng, greedy, rng.randint(1, 4), rng.choice([1, 2, 5, 16, 64]), 256, rng.choice([None, 3, 7]))
    params = [SamplingParams(max_new_tokens=m) for m in news]
    reqs = loop.run(prompts, params)
    for p, m, r in zip(prompts, news, reqs):
        assert r.output == [(len(p) + k) % VOCAB for k in range(m)]
    assert eng.cache.live == []
    eng.cache.check_invariants()


def test_prompts_that_advance_side_by_side_cannot_wedge_the_pool():
    """Portions smaller than the token budget let several prompts advance together; they can use the
    pool up while all of them are still mid-prompt, when no decoding request is there to preempt
    anybody.  The youngest then gives way: 10 pages of 16, two prompts of 128 tokens, budget 64,
    portions of 32 (each request alone fits: 128 + 7 tokens need 9 pages)."""
    eng = FakeEngine(num_pages=10, page_size=16, max_seqs=4)
    prompts = [[1] * 128, [1] * 128]
    reqs, _, loop = generate(prompts, max_new_tokens=8, engine=eng, budget=64, chunk=32)
    assert [r.output for r in reqs] == [[(128 + k) % VOCAB for k in range(8)]] * 2
    assert loop.scheduler.stats["preemptions"] >= 1
    assert reqs[0].preemptions == 0  # the oldest always gets on


@pytest.mark.parametrize("seed", range(40))
def test_random_portions_and_pools_always_finish(seed):
    """Random portion sizes, token budgets, pools that barely hold the longest request, and two
    groups of layers with different page sizes: every request finishes with the right tokens, and
    the books of the cache are right after every step (the fake engine checks them)."""
    rng = random.Random(1000 + seed)
    n = rng.randint(2, 9)
    prompts = [[1] * rng.randint(1, 90) for _ in range(n)]
    news = [rng.randint(1, 12) for _ in range(n)]
    longest = max(len(p) + m for p, m in zip(prompts, news))
    pages = [rng.choice([2, 4, 8, 16]) for _ in range(rng.choice([1, 1, 2]))]
    groups = [CacheGroupSpec(f"kv{g}", ((g, "mixer"),), 1, 4, 0, page_size=p) for g, p in enumerate(pages)]
    slack = rng.randint(0, 5)
    num_pages = {f"kv{g}": -(-longest // p) + slack for g, p in enumerate(pages)}
    eng = FakeEngine(num_pages=num_pages, page_size=pages[0], max_seqs=rng.randint(1, 4), groups=groups)
    loop = GenerationLoop(eng, greedy, rng.randint(1, 4), rng.choice([2, 5, 16, 64]), 256, rng.choice([None, 1, 3, 7, 32]))
    reqs = loop.run(prompts, [SamplingParams(max_new_tokens=m) for m in news])
    for p, m, r in zip(prompts, news, reqs):
        assert r.output == [(len(p) + k) % VOCAB for k in range(m)]
    assert eng.cache.live == []
    eng.cache.check_invariants()


def test_groups_with_different_page_sizes_are_counted_each_for_itself():
    """A group with pages of 16 and one with pages of 4: the small pages run out first, and the
    scheduler must see that although the first group has room."""
    groups = [CacheGroupSpec("kv0", ("a",), 1, 4, 0, page_size=16), CacheGroupSpec("kv1", ("b",), 1, 4, 0, page_size=4)]
    eng = FakeEngine(num_pages={"kv0": 8, "kv1": 12}, page_size=16, max_seqs=4, groups=groups)  # 128 and 48 tokens
    reqs, _, loop = generate([[1] * 20, [1] * 20], max_new_tokens=12, engine=eng)
    assert [r.output for r in reqs] == [[(20 + k) % VOCAB for k in range(12)]] * 2
    assert loop.scheduler.stats["preemptions"] >= 1  # 2 * 31 tokens do not fit 48 places
    with pytest.raises(ValueError, match="could never finish"):
        loop.scheduler.add("big", [1] * 40, SamplingParams(max_new_tokens=12))  # 51 tokens need 13 small pages


def test_sampling_counter_survives_preemption():
    """The sampler sees (seed, number of tokens generated so far): recomputation after a preemption
    asks for the same draws again."""
    asked = []

    def recording(logits, params, steps):
        asked.extend((p.seed, s) for p, s in zip(params, steps))
        return greedy(logits, params, steps)

    eng = FakeEngine(num_pages=6, page_size=4, max_seqs=2)
    loop = GenerationLoop(eng, recording, 2, 64, 256)
    loop.run([[1] * 6, [1] * 6], [SamplingParams(max_new_tokens=10, seed=s) for s in (11, 22)])
    assert loop.scheduler.stats["preemptions"] > 0
    for seed in (11, 22):
        steps = [s for sd, s in asked if sd == seed]
        assert steps == list(range(10))  # each draw asked for exactly once, in order


def test_the_short_cut_for_decode_steps_plans_what_the_rules_plan():
    """A step in which everybody decodes and nobody can join is planned without walking the rules;
    whenever that happens the rules are asked too (they change nothing in that case) and must say
    the same."""
    rng = random.Random(3)
    prompts = [[1] * rng.randint(1, 12) for _ in range(7)]
    eng = FakeEngine(num_pages=40, page_size=4, max_seqs=3)
    loop = GenerationLoop(eng, greedy, 3, 64, 256)
    sched = loop.scheduler
    rules, schedule = sched._schedule, sched.schedule
    state = {"by_rules": 0, "short_cuts": 0}

    def counted_rules():
        state["by_rules"] += 1
        return rules()

    def checked_schedule():
        before = state["by_rules"]
        plan = schedule()
        if state["by_rules"] == before:  # the short cut answered
            state["short_cuts"] += 1
            again = rules()
            assert [(e.request.rid, e.tokens, e.samples) for e in again.entries] == [(e.request.rid, e.tokens, e.samples) for e in plan.entries]
            assert not again.preempted
        return plan

    sched._schedule, sched.schedule = counted_rules, checked_schedule
    reqs = loop.run(prompts, [SamplingParams(max_new_tokens=rng.randint(2, 15)) for _ in prompts])
    assert all(r.finished for r in reqs) and state["short_cuts"] > 10 and state["by_rules"] >= 3


class AheadEngine(FakeEngine):
    """A fake engine that can prepare the next decode step as the real one does: it takes that
    step's pages early, and uses the preparation only for the very step it was made for."""

    def __init__(self, *a, **kw):
        super().__init__(*a, **kw)
        self._decoded = None
        self.prepared = self.used = 0

    def step(self, entries):
        out = super().step(entries)
        self._decoded = [e.rid for e in entries] if all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries) else None
        self._epoch = self.cache.epoch
        return out

    def prepare_decode(self):
        if self._decoded is None or self._epoch != self.cache.epoch:  # (requests came or went since)
            return None
        need = sum(self.cache.new_pages_needed(r, 1)[0] for r in self._decoded)
        if need > self.cache.free_pages():
            return None
        for r in self._decoded:
            self.cache.extend(r, 1)
        self.prepared += 1
        return (list(self._decoded), self.cache.epoch)

    def step_prepared(self, prepared, entries):
        rids, epoch = prepared
        if epoch != self.cache.epoch or [e.rid for e in entries] != rids:
            return None
        if any(len(e.tokens) != 1 or list(e.want) != [0] for e in entries):
            return None
        self.used += 1
        return self.step(entries)


class LaunchingSampler:
    def __call__(self, logits, params, steps):
        return greedy(logits, params, steps)

    def launch(self, logits, params, steps):
        return logits.argmax(-1)


@pytest.mark.parametrize("seed", range(8))
def test_preparing_the_next_decode_step_changes_no_decision(seed):
    """With an engine that prepares the next decode step during the current one (and takes its
    pages early) the loop runs the same steps, preempts the same requests and gives the same
    tokens as without; requests end on stop tokens and budgets, join late, and pools are tight."""
    rng = random.Random(100 + seed)
    n = rng.randint(3, 10)
    prompts = [[1] * rng.randint(1, 30) for _ in range(n)]
    news = [rng.randint(1, 24) for _ in range(n)]
    stops = [(rng.randrange(VOCAB),) if rng.random() < 0.5 else () for _ in range(n)]
    page = rng.choice([2, 4, 8])
    longest = max(len(p) + m for p, m in zip(prompts, news))
    pages, seqs, live = -(-longest // page) + rng.randint(0, 6), rng.randint(1, 4), rng.randint(1, 4)
    budget, chunk = rng.choice([4, 5, 16, 64]), rng.choice([None, 3, 7])
    runs = []
    for make, sampler, ahead in ((FakeEngine, greedy, False), (AheadEngine, LaunchingSampler(), True), (AheadEngine, LaunchingSampler(), False)):
        eng = make(num_pages=pages, page_size=page, max_seqs=seqs)
        loop = GenerationLoop(eng, sampler, live, budget, 256, chunk, look_ahead=ahead)
        reqs = loop.run(prompts, [SamplingParams(max_new_tokens=m, stop_token_ids=s) for m, s in zip(news, stops)])
        assert eng.cache.live == []
        eng.cache.check_invariants()
        calls = [[(rid[2], start, k) for rid, start, k in call] for call in eng.calls]
        runs.append(([r.output for r in reqs], [r.stop_reason for r in reqs], calls, loop.scheduler.stats["preemptions"]))
        if ahead:
            assert loop.stats["prepared_steps"] == eng.used
        elif make is AheadEngine:
            assert eng.prepared == 0
    assert runs[0] == runs[1] == runs[2]


def test_prepared_steps_are_used_and_dropped():
    """Two requests decode side by side: all their decode steps but the first run prepared, until
    one ends on its stop token; the step after that is planned anew."""
    eng = AheadEngine(num_pages=32, page_size=4, max_seqs=2)
    loop = GenerationLoop(eng, LaunchingSampler(), 2, 64, 256)
    reqs = loop.run([[1] * 3, [1] * 5], [SamplingParams(max_new_tokens=12, stop_token_ids=(9,)), SamplingParams(max_new_tokens=12)])
    assert reqs[0].output == [3, 4, 5, 6, 7, 8, 9] and len(reqs[1].output) == 12
    # steps: 1 prefill, 11 decode steps; prepared were all decode steps but the first one, the one
    # after the first request ended (its preparation no longer fits), and none after the last
    assert len(eng.calls) == 12
    assert eng.used == 11 - 2
    assert eng.prepared == eng.used + 1  # one was made in vain


# ----------------------------------------------------------------------------- steps launched ahead of the host
class LaunchAheadEngine(AheadEngine):
    """A fake engine that also runs a prepared step before the host has seen the tokens it is fed
    (they are "on the device": a tensor).  Like the real one it then runs a row for every request
    of the preparation, also for one that ends on that very token."""

    def __init__(self, *a, **kw):
        super().__init__(*a, **kw)
        self.launched = 0
        self.fed = []  # per launched step: (rid, position, token id fed)

    def step_prepared_on_device(self, prepared, rids, token_ids):
        from torchllms_amd.engine import StepEntry

        known, epoch = prepared
        if epoch != self.cache.epoch or list(rids) != known or token_ids.numel() != len(known):
            return None
        self.launched += 1
        self.used += 1
        self.fed.append([(rid, self.cache.num_tokens(rid), int(t)) for rid, t in zip(rids, token_ids)])
        return self.step([StepEntry(rid, [int(t)], [0]) for rid, t in zip(rids, token_ids)])


def _run(make, sampler, look_ahead, prompts, params, live=4, budget=64, chunk=None, **engine_kw):
    eng = make(**engine_kw)
    loop = GenerationLoop(eng, sampler, live, budget, 256, chunk, look_ahead=look_ahead)
    steps = []
    loop.launched_by_step = []  # steps launched ahead so far, as each step is booked

    def on_step(plan):
        steps.append([(e.request.rid[2], len(e.tokens)) for e in plan.entries])
        loop.launched_by_step.append(loop.stats["launched_ahead"])

    reqs = loop.run(prompts, params, on_step=on_step)
    assert eng.cache.live == [] and all(eng.cache.free_pages(g) == p.num_pages for g, p in enumerate(eng.cache.pools))
    eng.cache.check_invariants()
    return reqs, eng, loop, steps


@pytest.mark.parametrize("seed", range(12))
def test_steps_launched_ahead_give_the_same_tokens(seed):
    _launched_ahead_against_waiting(seed)


def _launched_ahead_against_waiting(seed):
    """Random workloads (stop tokens, budgets, late joiners, tight pools, preemptions) through the
    loop that launches the prepared step with the tokens still on the device, against the loop that
    waits before every step: the same tokens and stop reasons, every token fed ahead is the one
    that was sampled, and a request that ended on the token it was fed leaves nothing behind."""
    rng = random.Random(700 + seed)
    n = rng.randint(3, 10)
    prompts = [[1] * rng.randint(1, 30) for _ in range(n)]
    news = [rng.randint(1, 30) for _ in range(n)]
    stops = [(rng.randrange(VOCAB),) if rng.random() < 0.6 else () for _ in range(n)]
    page = rng.choice([2, 4, 8])
    longest = max(len(p) + m for p, m in zip(prompts, news))
    kw = dict(num_pages=-(-longest // page) + rng.randint(0, 6), page_size=page, max_seqs=rng.randint(1, 4))
    live, budget, chunk = rng.randint(1, 4), rng.choice([4, 5, 16, 64]), rng.choice([None, 3, 7])
    params = [SamplingParams(max_new_tokens=m, stop_token_ids=s) for m, s in zip(news, stops)]
    want, _, base, _ = _run(FakeEngine, greedy, False, prompts, params, live, budget, chunk, **kw)
    got, eng, loop, _ = _run(LaunchAheadEngine, LaunchingSampler(), True, prompts, params, live, budget, chunk, **kw)
    assert [r.output for r in got] == [r.output for r in want]
    assert [r.stop_reason for r in got] == [r.stop_reason for r in want]
    assert loop.stats["launched_ahead"] == eng.launched and loop.stats["prepared_steps"] == eng.used
    for step in eng.fed:
        for rid, pos, tok in step:
            assert tok == pos % VOCAB  # the token the fake model gives for the position before
    return loop.stats["launched_ahead"], loop.scheduler.stats["preemptions"], base.scheduler.stats["preemptions"]


def test_the_random_workloads_launch_ahead_and_preempt():
    """(The premise of the test above: among its workloads are some that launch steps ahead and
    preempt requests in the same run.)"""
    seen = [_launched_ahead_against_waiting(seed) for seed in range(12)]
    assert sum(1 for launched, preempted, _ in seen if launched > 3 and preempted > 0) >= 2, seen
    assert sum(launched for launched, _, _ in seen) > 50


def test_a_request_that_ends_on_the_token_it_was_fed_ahead():
    """Two requests decode side by side, steps launched ahead; the first ends on its stop token while
    the step that feeds that token to it is already running.  Its row is dropped, the other request's
    row of that step counts, and a third request that waited takes the seat one step later than in
    the loop that waits for the tokens."""
    prompts = [[1] * 3, [1] * 5, [1] * 2]
    params = [SamplingParams(max_new_tokens=12, stop_token_ids=(9,)), SamplingParams(max_new_tokens=12), SamplingParams(max_new_tokens=4)]
    want, _, _, base_steps = _run(FakeEngine, greedy, False, prompts, params, live=2, num_pages=32, page_size=4, max_seqs=2)
    got, eng, loop, steps = _run(LaunchAheadEngine, LaunchingSampler(), True, prompts, params, live=2, num_pages=32, page_size=4, max_seqs=2)
    assert [r.output for r in got] == [r.output for r in want]
    assert got[0].output == [3, 4, 5, 6, 7, 8, 9] and got[0].stop_reason == 9 and len(got[1].output) == 12
    # request 0 was fed its stop token (9, at position 9) by a step that was launched ahead
    assert any((rid[2], pos, tok) == (0, 9, 9) for step in eng.fed for rid, pos, tok in step)
    # that step counts for request 1 alone
    first = lambda all_steps: next(i for i, s in enumerate(all_steps) if any(r == 2 for r, _ in s))
    assert [0] not in [[r for r, _ in s] for s in steps] and [(1, 1)] in steps
    assert first(steps) == first(base_steps) + 1
    assert loop.stats["launched_ahead"] >= 8


def test_every_request_ends_on_the_token_that_was_fed_ahead():
    """Both requests end on the same step's token while the next step is already running for both:
    nothing of that step counts, nothing is left in the cache, and the loop ends."""
    prompts = [[1] * 4, [1] * 4]
    params = [SamplingParams(max_new_tokens=20, stop_token_ids=(11,)) for _ in prompts]
    got, eng, loop, steps = _run(LaunchAheadEngine, LaunchingSampler(), True, prompts, params, live=2, num_pages=16, page_size=4, max_seqs=2)
    assert [r.output for r in got] == [list(range(4, 12))] * 2 and [r.stop_reason for r in got] == [11, 11]
    assert eng.fed[-1] == [(r.rid, 11, 11) for r in got]  # the step in vain
    assert len(steps) == len(eng.calls) - 1  # ... which the loop never booked


def test_when_a_waiting_request_could_join_although_nobody_ends():
    """The rule that keeps steps from being launched ahead of the scheduler: a request that waits
    could be admitted while everybody else decodes on only if a seat is free and pages are there or
    may come back (a window gives pages back during decoding; nothing else does)."""
    def state(window, num_pages, max_seqs, prompts):
        eng = FakeEngine(num_pages=num_pages, page_size=4, max_seqs=max_seqs, window=window)
        sched = Scheduler(eng.cache, max_seqs, 64, 256)
        for i, p in enumerate(prompts):
            sched.add(i, [1] * p, SamplingParams(max_new_tokens=8))
        plan = sched.schedule()
        eng.step(plan.step_entries())
        sched.update(plan, [5] * sum(e.samples for e in plan.entries))
        return sched

    assert not state(0, 16, 2, [8, 8]).may_admit_before_a_request_ends()  # nobody waits
    assert not state(0, 16, 2, [8, 8, 8]).may_admit_before_a_request_ends()  # no seat
    sched = state(0, 4, 3, [8, 8, 8])
    assert len(sched.running) == 2 and sched.waiting and sched.cache.free_pages() == 0
    assert not sched.may_admit_before_a_request_ends()  # a seat, but no page, and none can come back
    sched = state(8, 4, 3, [8, 8, 8])
    assert len(sched.running) == 2 and sched.waiting and sched.cache.free_pages() == 0
    assert sched.may_admit_before_a_request_ends()  # the window will give pages back
    sched = state(0, 5, 3, [8, 8, 8])
    assert len(sched.running) == 3 and not sched.may_admit_before_a_request_ends()  # it has joined already


def test_nothing_is_launched_ahead_while_a_waiting_request_could_join():
    """While that rule says that somebody could join, the loop asks the scheduler before every step
    and launches nothing ahead: the steps are those of the loop that waits for the tokens.  A third
    request that waits for pages in a cache without a window, a seat being free, can only get them
    from a request that ends, and steps are launched ahead while it waits."""
    prompts = [[1] * 17, [1] * 17, [1] * 6]
    params = [SamplingParams(max_new_tokens=12), SamplingParams(max_new_tokens=12), SamplingParams(max_new_tokens=30)]
    kw = dict(live=3, budget=64, num_pages=4, page_size=16, max_seqs=3)  # two pages each for the first two: none is left
    want, _, _, base_steps = _run(FakeEngine, greedy, False, prompts, params, **kw)
    got, eng, loop, steps = _run(LaunchAheadEngine, LaunchingSampler(), True, prompts, params, **kw)
    assert [r.output for r in got] == [r.output for r in want]
    joined = next(i for i, s in enumerate(steps) if any(r == 2 for r, _ in s))
    assert loop.launched_by_step[joined] >= 5, (steps[:joined], loop.launched_by_step)

    eng = LaunchAheadEngine(num_pages=4, page_size=16, max_seqs=3)
    loop = GenerationLoop(eng, LaunchingSampler(), 3, 64, 256)
    loop.scheduler.may_admit_before_a_request_ends = lambda: bool(loop.scheduler.waiting)
    steps = []
    got = loop.run(prompts, params, on_step=lambda plan: steps.append(([(e.request.rid[2], len(e.tokens)) for e in plan.entries], loop.stats["launched_ahead"])))
    assert [r.output for r in got] == [r.output for r in want]
    joined = next(i for i, (s, _) in enumerate(steps) if any(r == 2 for r, _ in s))
    assert [s for s, _ in steps[: joined + 1]] == base_steps[: joined + 1]
    assert steps[joined][1] == 0 and loop.stats["launched_ahead"] > 10 and loop.stats["prepared_steps"] > loop.stats["launched_ahead"] + 5
