"""Builds replay traces: the same requests cut into steps in different ways.

A trace is a list of steps in the format ``bin/trace_run`` reads:
``{"step": n, "entries": [{"id", "tokens", "want"}], "end": [ids]}``.  Every schedule asks for the
logits at every position of every request, so results can be compared position by position.
"""

from __future__ import annotations

from typing import Dict, List, Sequence

PORTION_SIZES = [7, 2, 13, 3, 24, 2, 5, 31, 2, 9]


def whole(requests: Dict[str, Sequence[int]]) -> List[dict]:
    """Each request alone, all its tokens in one step."""
    steps = []
    for rid, toks in requests.items():
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": list(toks), "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def tail(requests: Dict[str, Sequence[int]], n_tail: int = 32) -> List[dict]:
    """Each request alone: all but the last ``n_tail`` tokens in one step, the rest one by one."""
    steps = []
    for rid, toks in requests.items():
        toks = list(toks)
        head = max(len(toks) - n_tail, 1)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        for i in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}], "end": []})
        steps[-1]["end"] = [rid]
    return steps


def portions(requests: Dict[str, Sequence[int]], sizes: Sequence[int] = PORTION_SIZES) -> List[dict]:
    """Each request alone, in consecutive portions of changing size, down to two tokens."""
    steps = []
    k = 0
    for rid, toks in requests.items():
        toks = list(toks)
        i = 0
        while i < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - i)
            k += 1
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[i : i + n], "want": list(range(n))}], "end": []})
            i += n
        steps[-1]["end"] = [rid]
    return steps


def mixed(requests: Dict[str, Sequence[int]], max_live: int = 4, prompt_frac: float = 0.6,
          sizes: Sequence[int] = PORTION_SIZES) -> List[dict]:
    """Up to ``max_live`` requests at a time.  Each is fed in portions of changing size up to
    ``prompt_frac`` of its length and one token a step after that, so steps hold portions of some
    requests beside single tokens of others; a request sits out every fifth step; as one ends the
    next starts, taking over its pages."""
    waiting = list(requests.items())
    live: List[dict] = []
    steps: List[dict] = []
    k = 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live.append({"id": rid, "toks": list(toks), "i": 0, "turn": 0, "cut": max(int(len(toks) * prompt_frac), 1)})
            break  # staggered: at most one joins per step
        entries, end = [], []
        for r in live:
            r["turn"] += 1
            if r["turn"] % 5 == 0 and len(live) > 1:
                continue  # left out of this step, goes on later
            if r["i"] < r["cut"]:
                n = min(sizes[k % len(sizes)], r["cut"] - r["i"])
                k += 1
            else:
                n = 1
            toks = r["toks"][r["i"] : r["i"] + n]
            entries.append({"id": r["id"], "tokens": toks, "want": list(range(len(toks)))})
            r["i"] += n
            if r["i"] >= len(r["toks"]):
                end.append(r["id"])
        live = [r for r in live if r["id"] not in end]
        steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps


def max_live_tokens(steps: List[dict], round_to: int = 64) -> int:
    """The most tokens live requests hold at any time, each request rounded up to ``round_to``."""
    held: Dict[str, int] = {}
    peak = 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return peak


def positions_of(steps: List[dict]):
    """For every step, the (request, position) of each wanted logits row, in output order."""
    held: Dict[str, int] = {}
    out = []
    for s in steps:
        rows = []
        for e in s["entries"]:
            base = held.get(e["id"], 0)
            rows.extend((e["id"], base + w) for w in e["want"])
            held[e["id"]] = base + len(e["tokens"])
        for rid in s["end"]:
            held.pop(rid, None)
        out.append(rows)
    return out
