"""Cache manager: keys and values in fixed-size pages with a block table per request, and
slots for per-request state of fixed size.

Layers whose needs are alike (same heads, head size, window, tokens per page and element type) form
a *group*.  A group owns a pool of pages; one page id addresses the same token range in every layer
of the group.  A request holds one block table per group (logical block -> page id); groups may
differ in page size, so their tables differ in length and their pools in the pages a step takes.  Pages go back to the pool
when the request ends and, in a group with a window, as soon as the window has passed them.

The bookkeeping is plain host code and runs without a GPU; the page tensors are optional so the
allocator can be tested alone.

What the reference's pool does and this one keeps: lazy allocation at claim, ceil-division page
counts, a free list that hands recently freed pages out again, reference counts with an error on
double release, and an invariant checker (reference: torchllms/models/paged_kv.py:271-350 claim /
extend, 298-327 refcounts, 797-843 invariants).  Different on purpose: allocation is
all-or-nothing and can be asked for beforehand (``can_extend``), requests have a recycled dense
slot, and pools exist per group.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch


class OutOfPages(RuntimeError):
    """A group's pool cannot hold the tokens asked for."""


class OutOfSlots(RuntimeError):
    """Every request slot is taken."""


@dataclass(frozen=True)
class CacheGroupSpec:
    """Layers (runs of the execution order) that share one page pool."""

    name: str
    run_ids: Tuple[Hashable, ...]  # keys of the cache entries (one per layer run and mixer) that live in this group
    num_kv_heads: int
    head_dim: int
    window: int = 0  # 0: all keys stay; w > 0: only the last w positions are read
    page_size: int = 0  # tokens per page; 0: the manager's default
    dtype: Optional[str] = None  # "float32" / "bfloat16"; None: the manager's default


@dataclass(frozen=True)
class StateSlotSpec:
    """Fixed-size per-request state of some runs: one tensor [runs, max_seqs, *shape]."""

    name: str
    run_ids: Tuple[Hashable, ...]
    shape: Tuple[int, ...]
    dtype: str = "float32"


def group_layers(needs: Sequence[Tuple[Hashable, object]]) -> Tuple[List[CacheGroupSpec], List[StateSlotSpec]]:
    """Group ``(cache entry key, need)`` pairs: KV needs by (heads, head size, window, page size,
    dtype), state needs by (shape, dtype).  ``need`` is a ``parts.base.KVNeed`` / ``StateNeed``
    (duck-typed) or None."""
    kv: Dict[tuple, List[Hashable]] = {}
    st: Dict[Tuple[Tuple[int, ...], str], List[Hashable]] = {}
    for run_id, need in needs:
        if need is None:
            continue
        if hasattr(need, "num_kv_heads"):
            form = (need.num_kv_heads, need.head_dim, need.window, int(getattr(need, "page_size", None) or 0),
                    getattr(need, "dtype", None))
            kv.setdefault(form, []).append(run_id)
        elif hasattr(need, "shape"):
            st.setdefault((tuple(need.shape), need.dtype), []).append(run_id)
        else:
            raise TypeError(f"cache entry {run_id}: unknown cache need {need!r}")
    groups = [
        CacheGroupSpec(name=f"kv{i}", run_ids=tuple(runs), num_kv_heads=h, head_dim=d, window=w, page_size=p, dtype=t)
        for i, ((h, d, w, p, t), runs) in enumerate(kv.items())
    ]
    states = [
        StateSlotSpec(name=f"state{i}", run_ids=tuple(runs), shape=shape, dtype=dtype)
        for i, ((shape, dtype), runs) in enumerate(st.items())
    ]
    return groups, states


class PagePool:
    """Free list and reference counts of one group's pages (host only)."""

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError(f"a page pool needs at least one page, got {num_pages}")
        self.num_pages = num_pages
        # popped from the end: page 0 is handed out first, freed pages are handed out again first
        self._free: List[int] = list(range(num_pages - 1, -1, -1))
        self._refcount: List[int] = [0] * num_pages

    @property
    def free_count(self) -> int:
        return len(self._free)

    def take(self, n: int) -> List[int]:
        if n > len(self._free):
            raise OutOfPages(f"asked for {n} pages, {len(self._free)} free of {self.num_pages}")
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._refcount[p] = 1
        return out

    def give_back(self, pages: Sequence[int]) -> None:
        for p in pages:
            if not 0 <= p < self.num_pages:
                raise ValueError(f"page {p} does not exist")
            if self._refcount[p] <= 0:
                raise RuntimeError(f"page {p} released twice")
            self._refcount[p] -= 1
            if self._refcount[p] == 0:
                self._free.append(p)

    def share(self, pages: Sequence[int]) -> None:
        for p in pages:
            if self._refcount[p] <= 0:
                raise RuntimeError(f"page {p} is not held, cannot be shared")
            self._refcount[p] += 1

    def refcount(self, page: int) -> int:
        return self._refcount[page]


@dataclass
class RequestEntry:
    slot: int
    num_tokens: int = 0  # tokens whose keys/values are (or are being) written
    reserved_tokens: int = 0  # tokens the block tables have room for
    # per group: logical block -> page id, -1 where a window has passed and the page went back
    block_tables: List[List[int]] = field(default_factory=list)
    first_live_block: List[int] = field(default_factory=list)
    # per group: the block table as an int32 array, rebuilt only after the table has changed
    table_arrays: List[Optional[np.ndarray]] = field(default_factory=list)


@dataclass
class KVLayerView:
    """What a mixer sees of the cache for one run: its layer's pages and its group."""

    group: int
    k_pages: torch.Tensor  # [num_pages, Hkv, page_size, dh]
    v_pages: torch.Tensor
    page_size: int
    writes: bool = True  # False when this run borrows another run's cache


@dataclass
class StateView:
    """Per-request state of one run: ``tensor[slot]`` belongs to the request in that slot."""

    tensor: torch.Tensor  # [max_seqs, *shape]


class CacheManager:
    def __init__(
        self,
        groups: Sequence[CacheGroupSpec],
        states: Sequence[StateSlotSpec],
        page_size: int,
        num_pages,
        max_seqs: int,
        dtype: torch.dtype = torch.float32,
        device: Optional[str] = None,
    ):
        """``page_size`` and ``dtype``: what a group has that names none of its own.  ``num_pages``:
        an int (every group) or a dict group name -> pages.  ``device`` None: bookkeeping only, no
        tensors."""
        if page_size <= 0 or max_seqs <= 0:
            raise ValueError("page_size and max_seqs must be positive")
        self.groups = list(groups)
        self.states = list(states)
        self.page_size = page_size
        #: tokens per page of every group
        self.page_sizes: List[int] = [g.page_size or page_size for g in self.groups]
        self.dtypes: List[torch.dtype] = [getattr(torch, g.dtype) if g.dtype else dtype for g in self.groups]
        if any(p <= 0 for p in self.page_sizes):
            raise ValueError(f"page sizes must be positive, got {self.page_sizes}")
        self.max_seqs = max_seqs
        self.dtype = dtype
        self.device = device
        self.pools: List[PagePool] = []
        for g in self.groups:
            n = num_pages[g.name] if isinstance(num_pages, dict) else num_pages
            self.pools.append(PagePool(int(n)))
        self._requests: Dict[Hashable, RequestEntry] = {}
        #: without a window no page is given back before its request ends
        self._windowed = any(g.window > 0 for g in self.groups)
        #: counts admissions, releases and truncations: a plan made at one epoch describes the same
        #: requests, slots and pages at the same epoch only
        self.epoch = 0
        self._free_slots: List[int] = list(range(max_seqs - 1, -1, -1))
        # cache entry key -> (group index, layer index inside the group) / (state index, layer index)
        self._run_to_kv: Dict[Hashable, Tuple[int, int]] = {}
        self._run_to_state: Dict[Hashable, Tuple[int, int]] = {}
        for gi, g in enumerate(self.groups):
            for li, run in enumerate(g.run_ids):
                self._run_to_kv[run] = (gi, li)
        for si, s in enumerate(self.states):
            for li, run in enumerate(s.run_ids):
                self._run_to_state[run] = (si, li)
        self.k_pages: List[Optional[torch.Tensor]] = []
        self.v_pages: List[Optional[torch.Tensor]] = []
        self.state_tensors: List[Optional[torch.Tensor]] = []
        if device is not None:
            for gi, (g, pool) in enumerate(zip(self.groups, self.pools)):
                shape = (len(g.run_ids), pool.num_pages, g.num_kv_heads, self.page_sizes[gi], g.head_dim)
                self.k_pages.append(torch.zeros(shape, dtype=self.dtypes[gi], device=device))
                self.v_pages.append(torch.zeros(shape, dtype=self.dtypes[gi], device=device))
            for s in self.states:
                shape = (len(s.run_ids), max_seqs, *s.shape)
                self.state_tensors.append(torch.zeros(shape, dtype=getattr(torch, s.dtype), device=device))
        self._views: Dict[Tuple[Hashable, bool], object] = {}

    # ------------------------------------------------------------------ sizes
    @staticmethod
    def bytes_per_token(groups: Sequence[CacheGroupSpec], dtype: torch.dtype) -> int:
        """Bytes one cached token costs summed over all groups (keys and values, every layer)."""
        total = 0
        for g in groups:
            elt = torch.empty(0, dtype=getattr(torch, g.dtype) if g.dtype else dtype).element_size()
            total += 2 * len(g.run_ids) * g.num_kv_heads * g.head_dim * elt
        return total

    @staticmethod
    def pages_for_tokens(groups: Sequence[CacheGroupSpec], page_size: int, n_tokens: int) -> Dict[str, int]:
        """Pages per group (by name) that hold ``n_tokens`` tokens, at least one each."""
        return {g.name: max(-(-n_tokens // (g.page_size or page_size)), 1) for g in groups}

    def blocks_for(self, n_tokens: int, group: int = 0) -> int:
        """Pages of ``group`` that ``n_tokens`` tokens of one request occupy."""
        page = self.page_sizes[group] if self.page_sizes else self.page_size
        return -(-n_tokens // page)

    # ------------------------------------------------------------------ requests
    def has(self, rid: Hashable) -> bool:
        return rid in self._requests

    @property
    def live(self) -> List[Hashable]:
        return list(self._requests)

    @property
    def free_slots(self) -> int:
        return len(self._free_slots)

    def free_pages(self, group: int = 0) -> int:
        return self.pools[group].free_count

    def admit(self, rid: Hashable) -> int:
        """Give ``rid`` a slot (no pages yet); its state rows are zeroed.  Returns the slot."""
        if rid in self._requests:
            raise ValueError(f"request {rid!r} is already live")
        if not self._free_slots:
            raise OutOfSlots(f"all {self.max_seqs} request slots are taken")
        slot = self._free_slots.pop()
        self.epoch += 1
        self._requests[rid] = RequestEntry(
            slot=slot,
            block_tables=[[] for _ in self.groups],
            first_live_block=[0 for _ in self.groups],
            table_arrays=[None for _ in self.groups],
        )
        for t in self.state_tensors:
            if t is not None:
                t[:, slot].zero_()
        return slot

    def get(self, rid: Hashable) -> Optional[RequestEntry]:
        """The live request's entry, or None."""
        return self._requests.get(rid)

    def entry(self, rid: Hashable) -> RequestEntry:
        try:
            return self._requests[rid]
        except KeyError:
            raise KeyError(f"request {rid!r} is not live") from None

    def num_tokens(self, rid: Hashable) -> int:
        return self.entry(rid).num_tokens

    def slot(self, rid: Hashable) -> int:
        return self.entry(rid).slot

    def block_table(self, rid: Hashable, group: int = 0) -> List[int]:
        return self.entry(rid).block_tables[group]

    def block_table_array(self, rid: Hashable, group: int = 0) -> np.ndarray:
        """The block table as a read-only int32 array (kept until the table changes: a step plan
        copies rows of it instead of converting a list every step)."""
        e = self.entry(rid)
        arr = e.table_arrays[group]
        if arr is None:
            arr = np.asarray(e.block_tables[group], dtype=np.int32)
            arr.setflags(write=False)
            e.table_arrays[group] = arr
        return arr

    # ------------------------------------------------------------------ pages
    def _first_needed_block(self, group: int, first_query_pos: int) -> int:
        """The lowest block a query at ``first_query_pos`` (or later) can still read."""
        w = self.groups[group].window
        if w <= 0:
            return 0
        lo = first_query_pos - w + 1
        return max(lo, 0) // self.page_sizes[group]

    def pages_short(self, rid: Hashable, n_new: int) -> Dict[int, int]:
        """Per group, how many pages are missing to take ``n_new`` more tokens (0 if it fits)."""
        e = self.entry(rid)
        out = {}
        for gi, pool in enumerate(self.pools):
            extra = max(self.blocks_for(e.num_tokens + n_new, gi) - len(e.block_tables[gi]), 0)
            out[gi] = max(extra - pool.free_count, 0)
        return out

    def new_pages_needed(self, rid: Hashable, n_new: int) -> List[int]:
        """Per group, the pages that taking ``n_new`` more tokens allocates."""
        e = self.entry(rid)
        total = e.num_tokens + n_new
        return [max(self.blocks_for(total, gi) - len(e.block_tables[gi]), 0) for gi in range(len(self.groups))]

    def pages_for_new_request(self, n_tokens: int) -> List[int]:
        """Per group, the pages that the first ``n_tokens`` tokens of a request take."""
        return [self.blocks_for(n_tokens, gi) for gi in range(len(self.groups))]

    def can_extend(self, rid: Hashable, n_new: int) -> bool:
        return all(v == 0 for v in self.pages_short(rid, n_new).values())

    def extend(self, rid: Hashable, n_new: int) -> int:
        """Make room for ``n_new`` more tokens in every group, or raise ``OutOfPages`` and change
        nothing.  Returns the position of the first new token."""
        if n_new < 0:
            raise ValueError("n_new must be >= 0")
        e = self.entry(rid)
        total = e.num_tokens + n_new
        if all(total <= len(bt) * page for bt, page in zip(e.block_tables, self.page_sizes)):
            # the pages it holds have room (most decode steps): nothing to take
            e.reserved_tokens = max(e.reserved_tokens, total)
            return e.num_tokens
        short = self.pages_short(rid, n_new)
        if any(short.values()):
            raise OutOfPages(
                f"request {rid!r}: {n_new} more tokens after {e.num_tokens} need pages a pool lacks "
                f"(missing per group: { {self.groups[g].name: s for g, s in short.items() if s} })"
            )
        for gi, pool in enumerate(self.pools):
            extra = self.blocks_for(total, gi) - len(e.block_tables[gi])
            if extra > 0:
                e.block_tables[gi].extend(pool.take(extra))
                e.table_arrays[gi] = None
        e.reserved_tokens = max(e.reserved_tokens, total)
        return e.num_tokens

    def advance(self, rid: Hashable, n_new: int) -> None:
        """``n_new`` tokens were written.  Pages a window has passed go back to their pool."""
        e = self.entry(rid)
        for bt, page in zip(e.block_tables, self.page_sizes):
            if e.num_tokens + n_new > len(bt) * page:
                raise RuntimeError(f"request {rid!r}: advancing past the pages it holds (extend first)")
        e.num_tokens += n_new
        if not self._windowed:
            return
        for gi, pool in enumerate(self.pools):
            first = min(self._first_needed_block(gi, e.num_tokens), len(e.block_tables[gi]))
            bt = e.block_tables[gi]
            passed = [bt[b] for b in range(e.first_live_block[gi], first) if bt[b] >= 0]
            if passed:
                pool.give_back(passed)
                for b in range(e.first_live_block[gi], first):
                    bt[b] = -1
                e.table_arrays[gi] = None
            e.first_live_block[gi] = max(e.first_live_block[gi], first)

    def truncate(self, rid: Hashable, num_tokens: int) -> None:
        """Drop tokens beyond ``num_tokens`` and give trailing pages back (reference:
        paged_kv.py:367-405 clamps rows after a padded prefill).  Not defined below a window's edge."""
        e = self.entry(rid)
        if not 0 <= num_tokens <= e.num_tokens:
            raise ValueError(f"cannot truncate request {rid!r} from {e.num_tokens} to {num_tokens} tokens")
        for gi, pool in enumerate(self.pools):
            bt = e.block_tables[gi]
            keep = self.blocks_for(num_tokens, gi)
            if keep < e.first_live_block[gi]:
                raise ValueError("cannot truncate into pages a window has already released")
            tail = [p for p in bt[keep:] if p >= 0]
            pool.give_back(tail)
            del bt[keep:]
            e.table_arrays[gi] = None
        e.num_tokens = num_tokens
        e.reserved_tokens = num_tokens
        self.epoch += 1

    def free(self, rid: Hashable) -> None:
        """The request ends: all its pages and its slot go back."""
        e = self._requests.pop(rid, None)
        if e is None:
            raise KeyError(f"request {rid!r} is not live (freed twice?)")
        self.epoch += 1
        for gi, pool in enumerate(self.pools):
            pool.give_back([p for p in e.block_tables[gi] if p >= 0])
        self._free_slots.append(e.slot)

    # ------------------------------------------------------------------ views for the model
    def kv_view(self, run_id: Hashable, writes: bool = True) -> KVLayerView:
        gi, li = self._run_to_kv[run_id]
        return KVLayerView(
            group=gi,
            k_pages=self.k_pages[gi][li],
            v_pages=self.v_pages[gi][li],
            page_size=self.page_sizes[gi],
            writes=writes,
        )

    def state_view(self, run_id: Hashable) -> StateView:
        si, li = self._run_to_state[run_id]
        return StateView(tensor=self.state_tensors[si][li])

    def view(self, key: Hashable, writes: bool = True):
        """What is held under the cache entry ``key``: a ``KVLayerView`` (``writes`` False for a run
        that borrows another run's entry), a ``StateView``, or None when the entry needs nothing.
        The views are made once and kept: the tensors they point at never move."""
        try:
            return self._views[(key, writes)]
        except KeyError:
            pass
        if key in self._run_to_kv:
            v = self.kv_view(key, writes)
        elif key in self._run_to_state:
            v = self.state_view(key)
        else:
            v = None
        self._views[(key, writes)] = v
        return v

    def view_for_run(self, run_id: Hashable, cache_from: Optional[Hashable] = None):
        return self.view(run_id if cache_from is None else cache_from, writes=cache_from is None)

    def gather_kv(self, rid: Hashable, run_id: Hashable) -> Tuple[torch.Tensor, torch.Tensor]:
        """Keys and values of a request in position order, [n, Hkv, dh] each (debugging, tests).
        Positions whose page a window released come back as zeros."""
        gi, li = self._run_to_kv[run_id]
        e = self.entry(rid)
        g = self.groups[gi]
        page_size = self.page_sizes[gi]
        n = e.num_tokens
        k = torch.zeros((n, g.num_kv_heads, g.head_dim), dtype=self.dtypes[gi], device=self.device)
        v = torch.zeros_like(k)
        for b, page in enumerate(e.block_tables[gi]):
            lo = b * page_size
            hi = min(lo + page_size, n)
            if page < 0 or lo >= n:
                continue
            k[lo:hi] = self.k_pages[gi][li, page, :, : hi - lo].transpose(0, 1)
            v[lo:hi] = self.v_pages[gi][li, page, :, : hi - lo].transpose(0, 1)
        return k, v

    # ------------------------------------------------------------------ invariants
    def check_invariants(self) -> None:
        """No page lost, held twice or free while held; block counts match token counts; slots
        are a partition (reference: paged_kv.py:797-843)."""
        for gi, pool in enumerate(self.pools):
            held: Dict[int, int] = {}
            for rid, e in self._requests.items():
                bt = e.block_tables[gi]
                if e.table_arrays[gi] is not None and e.table_arrays[gi].tolist() != bt:
                    raise AssertionError(f"{rid!r}: the cached array of group {gi}'s block table is stale")
                need = self.blocks_for(max(e.num_tokens, e.reserved_tokens), gi)
                if len(bt) < self.blocks_for(e.num_tokens, gi):
                    raise AssertionError(f"{rid!r}: {len(bt)} blocks for {e.num_tokens} tokens")
                if len(bt) > need:
                    raise AssertionError(f"{rid!r}: holds {len(bt)} blocks, needs at most {need}")
                for b, p in enumerate(bt):
                    if p < 0:
                        if b >= e.first_live_block[gi]:
                            raise AssertionError(f"{rid!r}: live block {b} has no page")
                        continue
                    if b < e.first_live_block[gi]:
                        raise AssertionError(f"{rid!r}: block {b} is behind the window but still holds page {p}")
                    held[p] = held.get(p, 0) + 1
            free = pool._free
            if len(set(free)) != len(free):
                raise AssertionError(f"group {gi}: a page is on the free list twice")
            overlap = set(free) & set(held)
            if overlap:
                raise AssertionError(f"group {gi}: pages {sorted(overlap)} are both free and held")
            if len(free) + len(held) != pool.num_pages:
                lost = set(range(pool.num_pages)) - set(free) - set(held)
                raise AssertionError(f"group {gi}: pages {sorted(lost)} are neither free nor held")
            for p, uses in held.items():
                if pool.refcount(p) != uses:
                    raise AssertionError(f"group {gi}: page {p} has refcount {pool.refcount(p)} but {uses} holders")
            for p in free:
                if pool.refcount(p) != 0:
                    raise AssertionError(f"group {gi}: free page {p} has refcount {pool.refcount(p)}")
        slots = [e.slot for e in self._requests.values()]
        if len(set(slots)) != len(slots):
            raise AssertionError("two requests share a slot")
        if set(slots) & set(self._free_slots):
            raise AssertionError("a slot is both free and taken")
        if len(slots) + len(self._free_slots) != self.max_seqs:
            raise AssertionError("a slot was lost")
