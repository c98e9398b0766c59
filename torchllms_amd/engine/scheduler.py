"""Continuous-batching scheduler: admits requests, cuts prompts into portions under a token
budget, decodes, finishes and frees, and decides what happens when pages run out.

The reference has no scheduler: it takes a list of prompts, sorts them by length, prefills each
static batch in one forward and decodes in lock step until all rows are done
(reference: torchllms/inference/llm.py:762-997, 1113-1141); when pages run out the request fails
(torchllms/models/paged_kv.py:285-289).  What is kept from it are the rules of finishing: any-of
stop ids with the stop token kept, the budget ``min(max_len - prompt_len, max_new_tokens)``, the
last sampled token never fed back (llm.py:489-494, 568, 905-908).

Every step is built in this order: one token for every request that is decoding; then further
portions of prompts already started; then new requests from the waiting queue, while slots, pages
and the token budget last.  Pages are counted before anything is committed.  When a decoding
request cannot get the page it needs, the most recently admitted running request is preempted:
its pages and slot are freed and it returns to the front of the waiting queue to be recomputed
from its prompt plus everything it has generated so far.  Its sampling counter is the number of
generated tokens, so its output is unchanged.  A request that could not fit into an empty pool
is refused when it is added.

The scheduler is plain host code; it touches the cache manager's bookkeeping only.
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Hashable, List, Optional, Sequence

from ..cache.manager import CacheManager
from ..sampling.params import SamplingParams
from .layout import StepEntry

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"


@dataclass(eq=False)  # a request is itself, not its field values: membership tests stay cheap
class Request:
    rid: Hashable
    prompt: List[int]
    params: SamplingParams
    budget: int  # tokens it may still generate in total
    output: List[int] = field(default_factory=list)
    state: str = WAITING
    num_computed: int = 0  # of prompt + output, how many tokens are in the cache
    stop_reason: Optional[int] = None  # the stop token id, or None when the budget ended it
    preemptions: int = 0
    arrival: int = 0

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    @property
    def last_token(self) -> int:
        return self.output[-1] if self.output else self.prompt[-1]

    def token_slice(self, lo: int, hi: int) -> List[int]:
        """``tokens[lo:hi]`` without putting prompt and output together first."""
        n = len(self.prompt)
        if hi <= n:
            return self.prompt[lo:hi]
        if lo >= n:
            return self.output[lo - n : hi - n]
        return self.prompt[lo:] + self.output[: hi - n]

    @property
    def remaining(self) -> int:
        """Tokens not yet in the cache (the last generated token included)."""
        return len(self.prompt) + len(self.output) - self.num_computed

    @property
    def finished(self) -> bool:
        return self.state == FINISHED


@dataclass(eq=False)
class ScheduledEntry:
    request: Request
    tokens: List[int]
    samples: bool  # the portion reaches the request's end: its last logits are sampled from


@dataclass
class StepPlan:
    entries: List[ScheduledEntry] = field(default_factory=list)
    preempted: List[Request] = field(default_factory=list)

    @property
    def n_tokens(self) -> int:
        return sum(len(e.tokens) for e in self.entries)

    def step_entries(self) -> List[StepEntry]:
        return [StepEntry(e.request.rid, e.tokens, [len(e.tokens) - 1] if e.samples else []) for e in self.entries]


class Scheduler:
    def __init__(
        self,
        cache: CacheManager,
        max_num_seqs: int,
        max_num_batched_tokens: int,
        max_model_len: int,
        prefill_chunk: Optional[int] = None,
    ):
        if max_num_batched_tokens < 1 or max_num_seqs < 1:
            raise ValueError("max_num_seqs and max_num_batched_tokens must be at least 1")
        self.cache = cache
        self.max_num_seqs = min(max_num_seqs, cache.max_seqs)
        self.max_num_batched_tokens = max_num_batched_tokens
        self.max_model_len = max_model_len
        self.prefill_chunk = prefill_chunk or max_num_batched_tokens
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []  # in order of admission
        self._arrivals = 0
        self.stats = {"steps": 0, "tokens": 0, "preemptions": 0, "finished": 0}

    # ------------------------------------------------------------------ intake
    def add(self, rid: Hashable, prompt: Sequence[int], params: SamplingParams) -> Request:
        """Queue a request.  Budget: ``min(max_model_len - len(prompt), max_new_tokens)``
        (reference: llm.py:489-494); below 1 the request finishes at once with no tokens."""
        prompt = [int(t) for t in prompt]
        if not prompt:
            raise ValueError(f"request {rid!r}: empty prompt")
        budget = self.max_model_len - len(prompt)
        if params.max_new_tokens is not None:
            budget = min(budget, params.max_new_tokens)
        req = Request(rid=rid, prompt=prompt, params=params, budget=max(budget, 0), arrival=self._arrivals)
        self._arrivals += 1
        if req.budget < 1:
            req.state = FINISHED
            return req
        # the longest it can get: all but the last generated token sit in the cache
        longest = len(prompt) + req.budget - 1
        for g, pool in enumerate(self.cache.pools):
            need = self._most_pages_held(g, longest)
            if need > pool.num_pages:
                raise ValueError(
                    f"request {rid!r}: {longest} tokens need {need} pages, "
                    f"the pool has {pool.num_pages}; it could never finish"
                )
        self.waiting.append(req)
        return req

    @property
    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def may_admit_before_a_request_ends(self) -> bool:
        """Could a request that waits be admitted while the running ones all go on decoding?  A
        seat must be free for it, and if it waits for pages, pages must be able to come back
        meanwhile: only a group with a window gives pages back while its requests decode; without
        one, the pages that are free now are all it can hope for.  (Whoever runs decode steps
        without asking ``schedule`` may do so while this is False.)"""
        if not self.waiting or len(self.running) >= self.max_num_seqs or self.cache.free_slots == 0:
            return False
        if any(g.window > 0 for g in self.cache.groups):
            return True
        return all(pool.free_count >= p for pool, p in zip(self.cache.pools, self.cache.pages_for_new_request(1)))

    def _most_pages_held(self, group: int, n_tokens: int) -> int:
        """The pages of ``group`` that a request of ``n_tokens`` cannot do without.  A group that
        keeps every key needs them all; a group with a window gives pages back as the window passes
        them, and a portion can be cut down to one token, so what it must hold at once are the
        pages that ``window`` keys touch (one more when they straddle a page's edge)."""
        whole = self.cache.blocks_for(n_tokens, group)
        window = self.cache.groups[group].window
        if window <= 0:
            return whole
        return min(whole, self.cache.blocks_for(window, group) + 1)

    # ------------------------------------------------------------------ planning
    def _pages_for(self, req: Request, n_new: int) -> List[int]:
        """Per group, the pages that ``n_new`` more tokens of ``req`` take."""
        if self.cache.has(req.rid):
            return self.cache.new_pages_needed(req.rid, n_new)
        return self.cache.pages_for_new_request(n_new)

    def _preempt(self, req: Request, plan: StepPlan) -> None:
        self.cache.free(req.rid)
        self.running.remove(req)
        req.state = WAITING
        req.num_computed = 0
        req.preemptions += 1
        self.stats["preemptions"] += 1
        self.waiting.appendleft(req)
        plan.preempted.append(req)

    def schedule(self) -> StepPlan:
        """Decide the next step.  Pages are counted here and taken by ``Engine.step``."""
        # The common step of a running batch: everybody decodes, nobody can join, and even if
        # every request opened a page in every group the pools would hold them.  The rules of
        # ``_schedule`` give exactly this plan then, after many more questions.
        running = self.running
        if (
            running and len(running) <= self.max_num_batched_tokens
            and all(pool.free_count >= len(running) for pool in self.cache.pools)
            and (not self.waiting or len(running) >= self.max_num_seqs or self.cache.free_slots == 0)
            and all(len(r.prompt) + len(r.output) - r.num_computed == 1 for r in running)
        ):
            return StepPlan(entries=[ScheduledEntry(r, [r.last_token], True) for r in running])
        return self._schedule()

    def _schedule(self) -> StepPlan:
        plan = StepPlan()
        while True:
            self._plan_stages(plan)
            if plan.entries or not self.running:
                break
            # Nothing fits although requests are running: several prompts advanced side by side
            # and used the pool up before any of them could decode.  The same rule as for a
            # decoding request that finds no page: the youngest gives way, so the oldest always
            # gets on.
            if len(self.running) == 1:
                break  # alone and still stuck: the pool cannot hold it (``add`` should have refused it)
            self._preempt(self.running[-1], plan)
        if not plan.entries and self.has_work:
            raise RuntimeError(
                "scheduler is stuck: work is queued but nothing fits (pool too small for the head of the queue?)"
            )
        return plan

    def _plan_stages(self, plan: StepPlan) -> None:
        budget = self.max_num_batched_tokens
        free = [pool.free_count for pool in self.cache.pools]

        def fits(pages: List[int]) -> bool:
            return all(f >= p for f, p in zip(free, pages))

        def take(pages: List[int]) -> None:
            for g, p in enumerate(pages):
                free[g] -= p

        # (1) one token for every decoding request, oldest first; make room by preempting the youngest
        decoding = [r for r in self.running if r.remaining == 1]
        i = 0
        while i < len(decoding) and budget > 0:
            req = decoding[i]
            if req.state != RUNNING:  # preempted a moment ago
                i += 1
                continue
            pages = self._pages_for(req, 1)
            while not fits(pages):
                victim = self.running[-1]
                was_planned = [e for e in plan.entries if e.request is victim]
                for e in was_planned:  # give back what this step had counted for it
                    plan.entries.remove(e)
                    budget += len(e.tokens)
                self._preempt(victim, plan)
                for g in range(len(free)):
                    free[g] = self.cache.pools[g].free_count
                for e in plan.entries:
                    take(self._pages_for(e.request, len(e.tokens)))
                if victim is req:
                    break
            if req.state == RUNNING:
                plan.entries.append(ScheduledEntry(req, [req.last_token], samples=True))
                take(pages)
                budget -= 1
            i += 1

        # (2) prompts already started, in order of admission
        planned = {id(e.request) for e in plan.entries}
        for req in self.running:
            if budget <= 0:
                break
            if req.remaining <= 1 or id(req) in planned:
                continue
            n = min(req.remaining, budget, self.prefill_chunk)
            while n > 0 and not fits(self._pages_for(req, n)):
                n = self._shrink(req, n, free)
            if n <= 0:
                continue
            self._add_portion(plan, req, n)
            take(self._pages_for(req, n))
            budget -= n

        # (3) new requests, first come first served; nothing overtakes the head of the queue
        while self.waiting and budget > 0 and len(self.running) < self.max_num_seqs and self.cache.free_slots > 0:
            req = self.waiting[0]
            if req in plan.preempted:
                break  # it lost its pages in this very step; it starts again in a later one
            n = min(req.remaining, budget, self.prefill_chunk)
            while n > 0 and not fits(self._pages_for(req, n)):
                n = self._shrink(req, n, free)
            if n <= 0:
                break
            self.waiting.popleft()
            self.cache.admit(req.rid)
            req.state = RUNNING
            self.running.append(req)
            self._add_portion(plan, req, n)
            take(self._pages_for(req, n))
            budget -= n

    def _shrink(self, req: Request, n: int, free: List[int]) -> int:
        """The largest portion below ``n`` that the free pages of every group hold (0: none)."""
        held = self.cache.num_tokens(req.rid) if self.cache.has(req.rid) else 0
        live = self.cache.get(req.rid)
        room = n - 1
        for g, page in enumerate(self.cache.page_sizes):
            have_blocks = len(live.block_tables[g]) if live is not None else 0
            room = min(room, (have_blocks + max(free[g], 0)) * page - held)
        return max(room, 0)

    def _add_portion(self, plan: StepPlan, req: Request, n: int) -> None:
        toks = req.token_slice(req.num_computed, req.num_computed + n)
        plan.entries.append(ScheduledEntry(req, toks, samples=(n == req.remaining)))

    # ------------------------------------------------------------------ after the step
    def update(self, plan: StepPlan, sampled: Sequence[int]) -> List[Request]:
        """Book the step: ``sampled`` holds one token for every entry with ``samples``, in order.
        Returns the requests that finished; their pages and slots are free again."""
        done: List[Request] = []
        it = iter(sampled)
        for e in plan.entries:
            req = e.request
            req.num_computed += len(e.tokens)
            if not e.samples:
                continue
            tok = int(next(it))
            req.output.append(tok)
            if tok in req.params.stop_token_ids:
                req.stop_reason = tok
                self._finish(req, done)
            elif len(req.output) >= req.budget:
                self._finish(req, done)
        self.stats["steps"] += 1
        self.stats["tokens"] += plan.n_tokens
        return done

    def _finish(self, req: Request, done: List[Request]) -> None:
        req.state = FINISHED
        self.running.remove(req)
        self.cache.free(req.rid)
        self.stats["finished"] += 1
        done.append(req)

    def abort(self, req: Request) -> None:
        """Drop a request wherever it is; what it holds is given back."""
        if req.state == RUNNING:
            self.running.remove(req)
            self.cache.free(req.rid)
        elif req.state == WAITING and req in self.waiting:
            self.waiting.remove(req)
        req.state = FINISHED
