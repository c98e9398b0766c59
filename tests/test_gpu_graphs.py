"""Decode steps replayed from HIP graphs give what eager steps give: several replays, with the
program's own eager work (prompt portions, other batch shapes) and synchronisations between them,
each checked against an engine that never records graphs."""

import pytest
import torch

from .helpers import TINY, make_folder, random_tokens

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "A"])
def test_graph_replays_match_eager_steps(tmp_path, name, dtype):
    from torchllms_amd.engine import Engine, StepEntry

    cfg = TINY[name]
    folder = make_folder(tmp_path / "m", cfg, seed=31, dtype=torch.bfloat16, sharpen=True)
    page = 16 if name == "B" else 8
    eager = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=64, max_seqs=4, use_graphs=False)
    graphed = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=64, max_seqs=4, use_graphs=True)
    assert eager.graphs is None and graphed.graphs is not None
    vocab = cfg["vocab_size"]
    toks = {r: random_tokens(100, vocab, 700 + i) for i, r in enumerate("abcd")}
    fed = {r: 0 for r in toks}

    def both(entries):
        outs = []
        for eng in (eager, graphed):
            for e in entries:
                if not eng.cache.has(e.rid):
                    eng.admit(e.rid)
            outs.append(eng.step(entries).float().cpu())
        torch.cuda.synchronize()
        return outs

    def take(r, n, want_last=True):
        t = toks[r][fed[r] : fed[r] + n]
        fed[r] += n
        return StepEntry(r, t, [n - 1] if want_last else [])

    def check(a, b, what):
        if dtype == "float32":
            assert torch.equal(a, b), what
        else:
            assert (a - b).abs().max().item() <= 2 ** -6 * max(a.abs().max().item(), 1.0), what

    a, b = both([take("a", 9), take("b", 20)])  # eager prompt portions
    check(a, b, "prefill")
    held = []
    for step in range(40):
        if step == 6:
            both([take("c", 13)])  # an eager step of another shape between replays
        if step == 17:
            both([take("d", 5), take("c", 1)])  # mixed: not a pure decode step, runs eagerly
        rows = ["a", "b"] + (["c"] if step >= 6 else []) + (["d"] if step >= 30 else [])
        a, b = both([take(r, 1) for r in rows])
        check(a, b, f"decode step {step} with {len(rows)} rows")
        held.append((a, b))
    assert sum(g.replays for g in graphed.graphs.graphs.values()) >= 25  # a shape runs eagerly until it has come back
    assert len(graphed.graphs.graphs) >= 3  # batch sizes 2, 3, 4
    # results handed out earlier were not overwritten by later replays
    for a, b in held:
        check(a, b, "held result")
    for eng in (eager, graphed):
        for r in toks:
            eng.free(r)
        eng.cache.check_invariants()


def test_context_cap_buckets():
    from torchllms_amd.engine.graphs import context_cap

    assert [context_cap(n) for n in (1, 512, 513, 768, 769, 1024, 2176, 5000, 6144, 6145, 8192)] == [512, 512, 768, 768, 1024, 1024, 3072, 6144, 6144, 8192, 8192]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prepared_decode_steps_match_plain_steps(tmp_path, dtype):
    """Decode steps prepared one step ahead (plan made and uploaded before the tokens are known)
    give the logits of steps planned when they run, across pages' edges and the context cap's
    step from 512 to 768, and a preparation that no longer fits is refused."""
    from torchllms_amd.engine import Engine, StepEntry

    cfg = TINY["B"]
    folder = make_folder(tmp_path / "m", cfg, seed=33, dtype=torch.bfloat16, sharpen=True)
    plain = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=160, max_seqs=4, max_model_len=1100, beyond_max_positions=True)
    ahead = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=160, max_seqs=4, max_model_len=1100, beyond_max_positions=True)
    vocab = cfg["vocab_size"]
    toks = {r: random_tokens(600, vocab, 900 + i) for i, r in enumerate("abc")}
    start = {"a": 470, "b": 23, "c": 7}
    for eng in (plain, ahead):
        for r in toks:
            eng.admit(r)
        eng.step([StepEntry(r, toks[r][: start[r]], []) for r in toks])
    used = 0
    prepared = None
    for step in range(70):
        entries = [StepEntry(r, [toks[r][start[r] + step]], [0]) for r in toks]
        want = plain.step(entries).float().cpu()
        got = ahead.step_prepared(prepared, entries) if prepared is not None else None
        used += got is not None
        if got is None:
            got = ahead.step(entries)
        prepared = ahead.prepare_decode()  # before the step's result is read, as the loop does
        got = got.float().cpu()
        if dtype == "float32":
            assert torch.equal(want, got), step
        else:
            assert (want - got).abs().max().item() <= 2 ** -6 * max(want.abs().max().item(), 1.0), step
    # a shape runs eagerly twice and is recorded at its third step; from then on every step is
    # prepared, but for the same three steps after request a passes 512 tokens
    assert used >= 70 - 2 * 4
    assert plain.cache.num_tokens("a") == ahead.cache.num_tokens("a") == 540
    # other entries than the prepared ones, or a request gone: refused, nothing run
    steps_before = ahead.steps_run
    assert prepared is not None
    two = [StepEntry(r, [1], [0]) for r in "ab"]
    assert ahead.step_prepared(prepared, two) is None
    swapped = [StepEntry(r, [1], [0]) for r in "bac"]
    assert ahead.step_prepared(prepared, swapped) is None
    unwanted = [StepEntry(r, [1], []) for r in "abc"]
    assert ahead.step_prepared(prepared, unwanted) is None
    ahead.free("c")
    assert ahead.step_prepared(prepared, [StepEntry(r, [1], [0]) for r in "abc"]) is None
    assert ahead.steps_run == steps_before
    assert ahead.prepare_decode() is None  # the last decode step's requests are not all there
    for eng in (plain, ahead):
        for r in toks:
            if eng.cache.has(r):
                eng.free(r)
        eng.cache.check_invariants()
        assert eng.cache.free_pages() == 160


def test_an_engine_of_other_sizes_can_be_built_after_steps_were_recorded(tmp_path):
    """Building a bfloat16 engine measures its product kernels in recorded graphs; that has to work
    after another engine has recorded decode steps (torch keeps capture state between graphs, and a
    capture inside inference mode followed by one outside it is refused)."""
    from torchllms_amd.engine import Engine, StepEntry

    first = Engine.from_folder(make_folder(tmp_path / "a", TINY["A"], seed=1), dtype="bfloat16", page_size=8, num_pages=16, max_seqs=2)
    first.admit("a")
    first.step([StepEntry("a", [1, 2, 3], [])])
    for t in range(6):
        first.step([StepEntry("a", [4 + t], [0])])
    assert any(g.graph is not None for g in first.graphs.graphs.values())
    other = dict(TINY["A"], hidden_size=72, intermediate_size=200, head_dim=16, vocab_size=264)  # sizes no other test has
    second = Engine.from_folder(make_folder(tmp_path / "b", other, seed=2), dtype="bfloat16", page_size=8, num_pages=16, max_seqs=2)
    second.admit("b")
    logits = second.step([StepEntry("b", [5, 6, 7], [2])])
    assert logits.shape == (1, 264) and bool(torch.isfinite(logits).all())
    for t in range(4):
        first.step([StepEntry("a", [20 + t], [0])])  # the first engine's recordings still replay
