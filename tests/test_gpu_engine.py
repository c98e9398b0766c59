"""The engine against the plain implementation, in 32-bit and in bfloat16: each request alone and
whole; most of it in one step and the last 32 tokens one by one; in portions of changing size down
to two tokens; and mixed, up to four live requests with so few pages that they are used again."""

import pytest
import torch

from . import schedules
from .helpers import PAGE_SIZE, TINY, make_folder, random_tokens, read_folder
from .plain import llama as plain

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [70, 41, 100, 35, 50, 33], "B": [66, 40, 130, 35, 90], "C": [45, 300, 37, 64, 120]}
FP32_ATOL = 2e-5


def run_trace(engine, steps):
    """Feed a trace through ``Engine.step``; returns {(request, position): logits row on the CPU}."""
    from torchllms_amd.engine import StepEntry

    out = {}
    rows = schedules.positions_of(steps)
    for s, where in zip(steps, rows):
        entries = []
        for e in s["entries"]:
            if not engine.cache.has(e["id"]):
                engine.admit(e["id"])
            entries.append(StepEntry(e["id"], e["tokens"], e["want"]))
        logits = engine.step(entries).cpu()
        assert logits.shape == (len(where), engine.vocab_size)
        for key, row in zip(where, logits):
            assert key not in out
            out[key] = row
        for rid in s["end"]:
            engine.free(rid)
        engine.cache.check_invariants()
    assert engine.cache.live == []
    assert all(p.free_count == p.num_pages for p in engine.cache.pools)
    return out


class Case:
    """One tiny configuration: its folder, requests, plain logits, and engines per dtype."""

    def __init__(self, name, tmp):
        from torchllms_amd.engine import Engine

        self.name = name
        cfg = TINY[name]
        self.folder = make_folder(tmp / name, cfg, seed=11, dtype=torch.bfloat16, norm_jitter=0.1, sharpen=True)
        self.cfg, self.weights = read_folder(self.folder)
        self.requests = {f"r{i}": random_tokens(n, cfg["vocab_size"], 100 + i) for i, n in enumerate(LENGTHS[name])}
        self.plain32 = {rid: plain.forward(self.weights, self.cfg, t, torch.float32) for rid, t in self.requests.items()}
        self.plain16 = {rid: plain.forward(self.weights, self.cfg, t, torch.bfloat16).float() for rid, t in self.requests.items()}
        self.traces = {
            "whole": schedules.whole(self.requests),
            "tail": schedules.tail(self.requests),
            "portions": schedules.portions(self.requests),
            "mixed": schedules.mixed(self.requests),
        }
        page = PAGE_SIZE[name]
        pool_tokens = max(schedules.max_live_tokens(t) for t in self.traces.values())
        self.engines = {
            dt: Engine.from_folder(self.folder, dtype=dt, page_size=page, num_pages=-(-pool_tokens // page), max_seqs=4)
            for dt in ("float32", "bfloat16")
        }
        self._results = {}

    def result(self, dtype, schedule):
        key = (dtype, schedule)
        if key not in self._results:
            self._results[key] = run_trace(self.engines[dtype], self.traces[schedule])
        return self._results[key]


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("models")
    return {name: Case(name, tmp) for name in TINY}


def _max_err(result, truth):
    worst, where = 0.0, None
    for (rid, pos), row in result.items():
        e = (row - truth[rid][pos]).abs().max().item()
        if e > worst:
            worst, where = e, (rid, pos)
    return worst, where


@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_float32_matches_the_plain_model(cases, name, schedule):
    case = cases[name]
    got = case.result("float32", schedule)
    assert len(got) == sum(len(t) for t in case.requests.values())
    err, where = _max_err(got, case.plain32)
    assert err < FP32_ATOL, f"{name}/{schedule}: first look at {where}, max abs error {err}"


@pytest.mark.parametrize("schedule", ["tail", "portions", "mixed"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_float32_does_not_depend_on_the_schedule(cases, name, schedule):
    """In 32-bit every kernel accumulates in an order fixed per output element, so logits are the
    same bits however the tokens were cut into steps, batched, or placed in pages."""
    case = cases[name]
    ref = case.result("float32", "whole")
    got = case.result("float32", schedule)
    diff = [k for k in ref if not torch.equal(ref[k], got[k])]
    assert not diff, f"{name}/{schedule}: {len(diff)} positions differ, first {sorted(diff)[0]}"


@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_bfloat16_is_as_close_as_plain_bfloat16(cases, name, schedule):
    """The yardstick for bfloat16 is the plain model run in bfloat16: the engine's distance from
    the 32-bit truth may not exceed twice the plain bfloat16 model's own, in the maximum, in the
    mean, and position by position (there against the plain model's error at that very position,
    or its mean over all positions where that is larger: a fault confined to one position, a page's
    edge say, does not hide below the largest error found anywhere)."""
    case = cases[name]
    got = case.result("bfloat16", schedule)
    ref_max = max((case.plain16[r] - case.plain32[r]).abs().max().item() for r in case.requests)
    ref_mean = torch.cat([(case.plain16[r] - case.plain32[r]).abs().flatten() for r in case.requests]).mean().item()
    err, where = _max_err(got, case.plain32)
    mean = torch.stack([(row - case.plain32[rid][pos]).abs().mean() for (rid, pos), row in got.items()]).mean().item()
    assert err <= 2 * ref_max, f"{name}/{schedule}: {where} max abs error {err} vs plain bfloat16 {ref_max}"
    assert mean <= 2 * ref_mean, f"{name}/{schedule}: mean abs error {mean} vs plain bfloat16 {ref_mean}"
    floor = torch.cat([(case.plain16[r] - case.plain32[r]).abs().amax(dim=1) for r in case.requests]).mean().item()
    for (rid, pos), row in got.items():
        here = (row - case.plain32[rid][pos]).abs().max().item()
        plain_here = (case.plain16[rid][pos] - case.plain32[rid][pos]).abs().max().item()
        assert here <= 2 * max(plain_here, floor), (
            f"{name}/{schedule}: {rid} position {pos}: error {here}, plain bfloat16 there {plain_here}, on average {floor}"
        )


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_bfloat16_schedules_agree(cases, name):
    case = cases[name]
    ref = case.result("bfloat16", "whole")
    ref_max = max((case.plain16[r] - case.plain32[r]).abs().max().item() for r in case.requests)
    for schedule in ("tail", "portions", "mixed"):
        got = case.result("bfloat16", schedule)
        err = max((ref[k] - got[k]).abs().max().item() for k in ref)
        assert err <= 2 * ref_max, f"{name}/{schedule} differs from whole by {err}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(cases, dtype):
    """Positions 0, 1, 2: a one-token step at position 0, then another, then a two-token portion."""
    from torchllms_amd.engine import StepEntry

    case = cases["B"]
    eng = case.engines[dtype]
    toks = case.requests["r0"]
    eng.admit("first")
    rows = [eng.step([StepEntry("first", toks[0:1], [0])]), eng.step([StepEntry("first", toks[1:2], [0])]),
            eng.step([StepEntry("first", toks[2:4], [0, 1])])]
    eng.free("first")
    got = torch.cat(rows).cpu()
    want = case.plain32["r0"][:4]
    tol = FP32_ATOL if dtype == "float32" else 2 * (case.plain16["r0"][:4] - want).abs().max().item()
    assert (got - want).abs().max().item() <= tol


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(cases, dtype):
    """A short prompt, then 280 tokens one by one: many pages, many steps."""
    from torchllms_amd.engine import StepEntry

    case = cases["C"]
    eng = case.engines[dtype]
    toks = case.requests["r1"]
    eng.admit("long")
    rows = [eng.step([StepEntry("long", toks[:20], [19])])]
    for i in range(20, len(toks)):
        rows.append(eng.step([StepEntry("long", toks[i : i + 1], [0])]))
    eng.free("long")
    got = torch.cat(rows).cpu()
    want = case.plain32["r1"][19:]
    tol = FP32_ATOL if dtype == "float32" else 2 * (case.plain16["r1"][19:] - want).abs().max().item()
    err = (got - want).abs().amax(dim=1)
    assert err.max().item() <= tol, f"first position over tolerance: {19 + int((err > tol).nonzero()[0])}"


def test_step_refuses_what_it_cannot_run(cases):
    from torchllms_amd.cache import OutOfPages
    from torchllms_amd.engine import StepEntry

    eng = cases["A"].engines["float32"]
    with pytest.raises(KeyError, match="not live"):
        eng.step([StepEntry("nobody", [1])])
    eng.admit("x")
    with pytest.raises(ValueError, match="outside the vocabulary"):
        eng.step([StepEntry("x", [256])])
    with pytest.raises(ValueError, match="twice"):
        eng.step([StepEntry("x", [1]), StepEntry("x", [2])])
    with pytest.raises(ValueError, match="max_model_len"):
        eng.step([StepEntry("x", [1] * 129)])
    eng.admit("y")
    eng.cache.admit("hog")
    eng.cache.extend("hog", (eng.cache.free_pages() - 1) * eng.page_size)  # one page is left
    with pytest.raises(OutOfPages):
        eng.step([StepEntry("x", [1, 2, 3]), StepEntry("y", [1] * (eng.page_size + 1))])
    assert eng.cache.free_pages() == 1 and eng.num_tokens("x") == 0 and eng.cache.block_table("x") == []
    eng.cache.free("hog")
    assert eng.step([StepEntry("x", [1, 2, 3])]).shape == (0, 256)  # nothing wanted
    eng.free("x")
    eng.free("y")
    eng.cache.check_invariants()


def test_decode_steps_planned_from_the_last_plan_equal_the_general_plan(cases):
    """A decode step that follows a decode step of the same requests is planned from that step's
    plan.  Both planners are run side by side on two engines through starts of pages, a request
    that ends, one that joins, a step with a prompt portion in between and a changed `want`."""
    import numpy as np

    from torchllms_amd.engine import Engine, StepEntry

    case = cases["B"]
    page = 4
    engines = [Engine.from_folder(case.folder, dtype="float32", page_size=page, num_pages=64, max_seqs=4, use_graphs=False) for _ in range(2)]
    fast, general = engines
    rng = torch.Generator().manual_seed(5)

    def both(entries):
        general._last_decode = None  # this engine always plans from scratch
        la, lb = fast.plan(entries), general.plan(entries)
        for name in ("tokens", "positions", "token_seq", "qo_indptr", "kv_lens", "slot_ids", "logit_rows"):
            assert np.array_equal(getattr(la, name), getattr(lb, name)), name
        assert (la.n_tokens, la.n_seqs, la.n_decode, la.max_q_len, la.max_kv_len) == (lb.n_tokens, lb.n_seqs, lb.n_decode, lb.max_q_len, lb.max_kv_len)
        for g in range(len(la.block_tables)):
            assert np.array_equal(la.slot_mappings[g], lb.slot_mappings[g])
            wa, wb = la.block_tables[g].shape[1], lb.block_tables[g].shape[1]
            w = min(wa, wb)
            assert np.array_equal(la.block_tables[g][:, :w], lb.block_tables[g][:, :w])
            assert (la.block_tables[g][:, w:] == -1).all() and (lb.block_tables[g][:, w:] == -1).all()
        for eng in engines:
            for e in entries:
                eng.cache.advance(e.rid, len(e.tokens))
        return la

    def tok():
        return int(torch.randint(0, case.cfg["vocab_size"], (1,), generator=rng))

    for eng in engines:
        for rid in ("a", "b", "c"):
            eng.admit(rid)
    both([StepEntry("a", [tok() for _ in range(5)], [4]), StepEntry("b", [tok() for _ in range(3)], [2]), StepEntry("c", [tok()], [0])])
    used_fast = 0
    for step in range(30):
        live = ["a", "b", "c"] if step < 12 else (["a", "c"] if step < 20 else ["a", "c", "d"])
        if step == 12:
            for eng in engines:
                eng.free("b")
        if step == 20:
            for eng in engines:
                eng.admit("d")
            both([StepEntry("d", [tok(), tok()], [1])])
        want = [] if step == 7 else [0]
        before = fast._last_decode
        layout = both([StepEntry(r, [tok()], want) for r in live])
        used_fast += before is not None and fast._last_decode is not None and fast._last_decode[2] is layout and before[0] == tuple(live)
    assert used_fast >= 15  # the shortcut did plan most of these steps
    for eng in engines:
        eng.cache.check_invariants()


def test_pool_sizes(cases):
    """The pool is as large as asked: pages, gigabytes, a fraction of free memory, or room for
    ``max_seqs`` requests of ``max_model_len`` tokens."""
    from torchllms_amd.cache import CacheManager
    from torchllms_amd.engine import Engine

    folder = cases["A"].folder
    per_page = None
    for kw, check in [
        (dict(num_pages=7), lambda n, pp: n == 7),
        (dict(kv_memory_gb=1 / 1024), lambda n, pp: n == (1 << 20) // pp),
        (dict(kv_memory_fraction=1e-4), lambda n, pp: 1 <= n <= torch.cuda.mem_get_info()[1] * 1e-4 // pp),
        (dict(max_seqs=3, max_model_len=50), lambda n, pp: n == 3 * 7),
    ]:
        eng = Engine.from_folder(folder, dtype="float32", page_size=8, **kw)
        per_page = 8 * CacheManager.bytes_per_token(eng.cache.groups, torch.float32)
        assert check(eng.cache.pools[0].num_pages, per_page), kw
    with pytest.raises(ValueError, match="kv_memory_fraction"):
        Engine.from_folder(folder, dtype="float32", kv_memory_fraction=1.5)


def test_sizes_no_kernel_takes_are_refused_when_the_engine_is_built():
    """Not at the first step: ``Engine`` asks every part at construction, before it loads anything."""
    from torchllms_amd.config import LlamaConfig
    from torchllms_amd.engine import Engine

    cfg = LlamaConfig.from_dict(dict(TINY["B"], head_dim=272, num_hidden_layers=1))
    for dtype in ("float32", "bfloat16"):
        with pytest.raises(ValueError, match="head size 272.*up to 256"):
            Engine.from_random(cfg, seed=0, dtype=dtype, max_seqs=1, max_model_len=64)
    cfg = LlamaConfig.from_dict(dict(TINY["B"], head_dim=256, num_hidden_layers=1))
    eng = Engine.from_random(cfg, seed=0, dtype="bfloat16", max_seqs=1, max_model_len=64)
    with pytest.raises(ValueError, match="page_size"):
        Engine.from_random(cfg, seed=0, dtype="bfloat16", max_seqs=1, max_model_len=64, page_size=0)
    del eng


def test_a_context_longer_than_the_models_positions_is_refused_unless_asked_for(cases):
    """The reference's table of angles ends at ``max_position_embeddings`` and a longer request fails
    there (reference: networks.py:325-327).  Here angles come from positions, so it would run: the
    engine refuses such a ``max_model_len`` unless told to go beyond, and ``LLM`` takes its ``max_len``
    as a bound beside the model's own."""
    from torchllms_amd.engine import Engine, StepEntry
    from torchllms_amd.inference import LLM

    folder = cases["A"].folder  # 128 positions
    with pytest.raises(ValueError, match="max_model_len=129 exceeds the 128 positions"):
        Engine.from_folder(folder, dtype="float32", max_seqs=1, max_model_len=129)
    assert Engine.from_folder(folder, dtype="float32", max_seqs=1).max_model_len == 128
    eng = Engine.from_folder(folder, dtype="float32", max_seqs=1, max_model_len=140, beyond_max_positions=True)
    eng.admit("r")
    assert eng.step([StepEntry("r", random_tokens(135, 256, 1), [134])]).shape == (1, 256)
    assert LLM(str(folder), precision="float32", max_len=4096, max_bsz=1).max_len == 128


def test_a_step_that_fails_leaves_nothing_behind(cases):
    """A step whose forward pass raises books nothing: the pages it took go back, the request is
    where it was, and the next step is planned afresh."""
    from torchllms_amd.engine import Engine, StepEntry

    eng = Engine.from_folder(cases["A"].folder, dtype="float32", page_size=8, num_pages=12, max_seqs=2, use_graphs=False)
    eng.admit("r")
    first = eng.step([StepEntry("r", [1, 2, 3, 4, 5], [4])]).cpu()
    free = eng.cache.free_pages()
    real_forward = eng.model.forward
    eng.model.forward = lambda ctx, cache: (_ for _ in ()).throw(RuntimeError("kernel failed"))
    for tokens in ([7], list(range(30))):
        with pytest.raises(RuntimeError, match="kernel failed"):
            eng.step([StepEntry("r", tokens, [0])])
        assert eng.num_tokens("r") == 5 and eng.cache.free_pages() == free and eng._last_decode is None
        eng.cache.check_invariants()
    eng.model.forward = real_forward
    again = eng.step([StepEntry("r", [7], [0])]).cpu()
    eng.free("r")
    eng.admit("s")
    whole = eng.step([StepEntry("s", [1, 2, 3, 4, 5, 7], [4, 5])]).cpu()
    eng.free("s")
    assert torch.equal(whole[0], first[0]) and torch.equal(whole[1], again[0])
