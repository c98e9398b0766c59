"""Host-side plan of one step: which tokens run, where they sit in their requests, where their
keys and values go, and which rows' logits are wanted.

The plan is a handful of int32 vectors packed into one buffer, so a step costs one host-to-device
copy.  The reference builds the same quantities per forward in ``build_batch_layout``
(reference: torchllms/models/paged_kv.py:486-617: qo_indptr, kv_indptr, kv_indices,
kv_last_page_len, batch_indices, positions); here block tables are a dense [rows, max_blocks]
matrix per group and the page/offset of each new token is precomputed as ``slot_mapping``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable, List, Sequence

import numpy as np


@dataclass
class StepEntry:
    """One request's share of a step: its next tokens and the places among them whose logits
    are wanted (indices into ``tokens``; empty: none)."""

    rid: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class StepLayout:
    """Everything about a step that is known on the host.  Rows with a single token come first
    (``n_decode`` of them) so that decode and prefill kernels each see a contiguous range."""

    n_tokens: int
    n_seqs: int
    n_decode: int
    row_of_entry: List[int]  # entry index -> row
    tokens: np.ndarray  # int32 [T]
    positions: np.ndarray  # int32 [T]
    token_seq: np.ndarray  # int32 [T]  row of each token
    qo_indptr: np.ndarray  # int32 [B + 1]
    kv_lens: np.ndarray  # int32 [B]  tokens of the row's request after this step
    slot_ids: np.ndarray  # int32 [B]  request slot of each row
    logit_rows: np.ndarray  # int32 [n_out]  flat token index of every wanted logit, in entry order
    block_tables: List[np.ndarray] = field(default_factory=list)  # per group int32 [B, max_blocks]
    slot_mappings: List[np.ndarray] = field(default_factory=list)  # per group int32 [T]
    page_sizes: List[int] = field(default_factory=list)  # per group, tokens per page
    max_q_len: int = 0
    max_kv_len: int = 0

    @property
    def decode_uneven(self) -> bool:
        """Whether the single-token rows differ much in context length: the longest holds more
        than one and a half times the mean.  The decode attention kernel then cuts the keys into
        shorter splits, so that the blocks of long requests spread over the CUs that short
        requests leave early."""
        n = self.n_decode
        if n < 2:
            return False
        lens = self.kv_lens[:n]
        return 2 * n * int(lens.max()) > 3 * int(lens.sum())

    @property
    def page_size(self) -> int:
        """Tokens per page of the first group."""
        return self.page_sizes[0] if self.page_sizes else 0

    # the reference's names for the same facts (of the first group), for comparison with its test vectors
    @property
    def kv_indptr(self) -> List[int]:
        out = [0]
        for n in self.kv_lens.tolist():
            out.append(out[-1] + -(-n // self.page_size))
        return out

    @property
    def kv_last_page_len(self) -> List[int]:
        return [((n - 1) % self.page_size) + 1 if n > 0 else 0 for n in self.kv_lens.tolist()]


def build_step_layout(
    entries: Sequence[StepEntry],
    starts: Sequence[int],
    slots: Sequence[int],
    block_tables: Sequence[Sequence[Sequence[int]]],
    page_size,
    decode_first: bool = True,
) -> StepLayout:
    """``starts[i]``: tokens entry i's request already holds; ``slots[i]``: its request slot;
    ``block_tables[g][i]``: its block table in group g, already long enough for the new tokens;
    ``page_size``: tokens per page, one number for all groups or a list with one per group."""
    page_sizes = [int(page_size)] * len(block_tables) if isinstance(page_size, int) else [int(p) for p in page_size]
    if len(page_sizes) != len(block_tables):
        raise ValueError(f"{len(block_tables)} groups of block tables, {len(page_sizes)} page sizes")
    n_entries = len(entries)
    order = list(range(n_entries))
    if decode_first:
        order.sort(key=lambda i: 0 if len(entries[i].tokens) == 1 else 1)  # stable
    row_of_entry = [0] * n_entries
    for row, i in enumerate(order):
        row_of_entry[i] = row
    n_decode = sum(1 for e in entries if len(e.tokens) == 1) if decode_first else 0

    q_lens = [len(entries[i].tokens) for i in order]
    if any(q <= 0 for q in q_lens):
        raise ValueError("every entry of a step needs at least one token")
    T = sum(q_lens)
    B = n_entries
    qo_indptr = np.zeros(B + 1, dtype=np.int32)
    np.cumsum(q_lens, out=qo_indptr[1:])
    tokens = np.empty(T, dtype=np.int32)
    positions = np.empty(T, dtype=np.int32)
    token_seq = np.empty(T, dtype=np.int32)
    kv_lens = np.empty(B, dtype=np.int32)
    slot_ids = np.empty(B, dtype=np.int32)
    bounds = qo_indptr.tolist()
    for row, i in enumerate(order):
        lo, hi = bounds[row], bounds[row + 1]
        if hi - lo == 1:  # a decoded token: scalars, no small arrays
            tokens[lo] = entries[i].tokens[0]
            positions[lo] = starts[i]
            token_seq[lo] = row
        else:
            tokens[lo:hi] = np.asarray(entries[i].tokens, dtype=np.int64)
            positions[lo:hi] = np.arange(starts[i], starts[i] + (hi - lo), dtype=np.int32)
            token_seq[lo:hi] = row
        kv_lens[row] = starts[i] + (hi - lo)
        slot_ids[row] = slots[i]

    logit_rows: List[int] = []
    for i, e in enumerate(entries):
        base = bounds[row_of_entry[i]]
        n = len(e.tokens)
        for w in e.want:
            if not 0 <= w < n:
                raise ValueError(f"request {e.rid!r}: wanted place {w} outside its {n} tokens")
            logit_rows.append(base + int(w))

    bts: List[np.ndarray] = []
    sms: List[np.ndarray] = []
    for g in range(len(block_tables)):
        page_size = page_sizes[g]
        max_blocks = max((len(block_tables[g][i]) for i in range(n_entries)), default=1)
        max_blocks = max(max_blocks, 1)
        bt = np.full((B, max_blocks), -1, dtype=np.int32)
        sm = np.empty(T, dtype=np.int32)
        for row, i in enumerate(order):
            table = np.asarray(block_tables[g][i], dtype=np.int32)
            bt[row, : len(table)] = table
            lo, hi = bounds[row], bounds[row + 1]
            if hi - lo == 1:
                page = int(table[starts[i] // page_size])
                if page < 0:
                    raise RuntimeError(f"request {entries[i].rid!r}: a new token has no page (extend first)")
                sm[lo] = page * page_size + starts[i] % page_size
                continue
            pos = positions[lo:hi]
            pages = table[pos // page_size]
            if (pages < 0).any():
                raise RuntimeError(f"request {entries[i].rid!r}: a new token has no page (extend first)")
            sm[lo:hi] = pages * page_size + pos % page_size
        bts.append(bt)
        sms.append(sm)

    return StepLayout(
        n_tokens=T,
        n_seqs=B,
        n_decode=n_decode,
        row_of_entry=row_of_entry,
        tokens=tokens,
        positions=positions,
        token_seq=token_seq,
        qo_indptr=qo_indptr,
        kv_lens=kv_lens,
        slot_ids=slot_ids,
        logit_rows=np.asarray(logit_rows, dtype=np.int32),
        block_tables=bts,
        slot_mappings=sms,
        page_sizes=page_sizes,
        max_q_len=max(q_lens) if q_lens else 0,
        max_kv_len=int(kv_lens.max()) if B else 0,
    )
