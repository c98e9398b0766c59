"""The trace builders themselves (CPU)."""

from .schedules import max_live_tokens, mixed, portions, positions_of, tail, whole


def _reqs():
    return {"a": list(range(70)), "b": list(range(100, 141)), "c": list(range(200, 290)), "d": list(range(35)), "e": list(range(50))}


def _covered(steps, reqs):
    seen = {}
    for rows, s in zip(positions_of(steps), steps):
        toks = [t for e in s["entries"] for t, _ in zip([e["tokens"][w] for w in e["want"]], e["want"])]
        for (rid, pos), tok in zip(rows, toks):
            assert (rid, pos) not in seen
            seen[(rid, pos)] = tok
    for rid, t in reqs.items():
        assert [seen[(rid, p)] for p in range(len(t))] == list(t)


def test_every_schedule_feeds_every_token_once():
    reqs = _reqs()
    for build in (whole, tail, portions, mixed):
        _covered(build(reqs), reqs)


def test_shapes_of_the_schedules():
    reqs = _reqs()
    t = tail({"a": reqs["a"]})
    assert len(t) == 33 and len(t[0]["entries"][0]["tokens"]) == 38
    p = portions({"a": reqs["a"]})
    assert min(len(s["entries"][0]["tokens"]) for s in p) == 2
    m = mixed(reqs)
    assert max(len(s["entries"]) for s in m) == 4
    assert any(len({len(e["tokens"]) == 1 for e in s["entries"]}) == 2 for s in m)  # portions beside single tokens
    assert max_live_tokens(m) < sum(-(-len(t) // 64) * 64 for t in reqs.values())  # so pages get used again
