"""The step's host-side plan (CPU).  Vectors marked (ref) restate
reference: torchllms/models/test_paged_kv.py:144-186."""

import pytest

from torchllms_amd.cache import CacheGroupSpec, CacheManager
from torchllms_amd.engine.layout import StepEntry, build_step_layout


def _plan(cache, entries, decode_first=False):
    starts = [cache.extend(e.rid, len(e.tokens)) for e in entries]
    slots = [cache.slot(e.rid) for e in entries]
    tables = [[cache.block_table(e.rid, 0) for e in entries]]
    lay = build_step_layout(entries, starts, slots, tables, cache.page_size, decode_first=decode_first)
    for e in entries:
        cache.advance(e.rid, len(e.tokens))
    return lay


def _cache():
    c = CacheManager([CacheGroupSpec("kv0", (0,), 2, 8)], [], page_size=4, num_pages=16, max_seqs=4)
    c.admit("r1")
    c.admit("r2")
    return c


def test_uniform_prefill():  # (ref)
    lay = _plan(_cache(), [StepEntry("r1", [1] * 5), StepEntry("r2", [2] * 5)])
    assert lay.n_seqs == 2 and lay.n_tokens == 10
    assert lay.qo_indptr.tolist() == [0, 5, 10]
    assert lay.kv_indptr == [0, 2, 4]
    assert lay.kv_last_page_len == [1, 1]
    assert lay.token_seq.tolist() == [0] * 5 + [1] * 5
    assert lay.positions.tolist() == list(range(5)) * 2


def test_decode_after_prefill():  # (ref)
    c = _cache()
    _plan(c, [StepEntry("r1", [1] * 5), StepEntry("r2", [2] * 3)])
    lay = _plan(c, [StepEntry("r1", [7]), StepEntry("r2", [8])])
    assert lay.qo_indptr.tolist() == [0, 1, 2]
    assert lay.kv_indptr == [0, 2, 3]
    assert lay.kv_last_page_len == [2, 4]
    assert lay.token_seq.tolist() == [0, 1]
    assert lay.positions.tolist() == [5, 3]


def test_ragged():  # (ref)
    lay = _plan(_cache(), [StepEntry("r1", [1] * 3), StepEntry("r2", [2] * 5)])
    assert lay.qo_indptr.tolist() == [0, 3, 8]
    assert lay.token_seq.tolist() == [0, 0, 0, 1, 1, 1, 1, 1]
    assert lay.positions.tolist() == [0, 1, 2, 0, 1, 2, 3, 4]


def test_slot_mapping_block_tables_and_wanted_rows():
    c = _cache()
    _plan(c, [StepEntry("r1", [1] * 6)])
    # a mixed step: a portion of r2's prompt beside one decoded token of r1; decode rows go first
    lay = _plan(c, [StepEntry("r2", [5, 6, 7], want=[2]), StepEntry("r1", [9], want=[0])], decode_first=True)
    assert lay.n_decode == 1 and lay.row_of_entry == [1, 0]
    assert lay.tokens.tolist() == [9, 5, 6, 7]
    assert lay.positions.tolist() == [6, 0, 1, 2]
    assert lay.kv_lens.tolist() == [7, 3]
    assert lay.logit_rows.tolist() == [3, 0]  # order of the entries as given, not of the rows
    bt1, bt2 = c.block_table("r1"), c.block_table("r2")
    assert lay.block_tables[0].tolist() == [bt1, bt2 + [-1]]
    assert lay.slot_mappings[0].tolist() == [bt1[1] * 4 + 2, bt2[0] * 4 + 0, bt2[0] * 4 + 1, bt2[0] * 4 + 2]
    assert lay.slot_ids.tolist() == [c.slot("r1"), c.slot("r2")]
    assert lay.max_q_len == 3 and lay.max_kv_len == 7


def test_bad_entries():
    c = _cache()
    with pytest.raises(ValueError, match="at least one token"):
        build_step_layout([StepEntry("r1", [])], [0], [0], [[[]]], 4)
    c.extend("r1", 2)
    with pytest.raises(ValueError, match="wanted place 2"):
        build_step_layout([StepEntry("r1", [1, 2], want=[2])], [0], [0], [[c.block_table("r1")]], 4)
    with pytest.raises(IndexError):
        build_step_layout([StepEntry("r1", [1] * 9)], [0], [0], [[c.block_table("r1")]], 4)


def test_decode_rows_of_unequal_length_are_told_apart():
    c = CacheManager([CacheGroupSpec("kv0", (0,), 2, 8)], [], page_size=4, num_pages=64, max_seqs=4)
    for rid, n in (("a", 40), ("b", 44), ("c", 36)):
        c.admit(rid)
        c.extend(rid, n)
        c.advance(rid, n)
    lay = _plan(c, [StepEntry(r, [1], want=[0]) for r in "abc"], decode_first=True)
    assert lay.kv_lens.tolist() == [41, 45, 37] and not lay.decode_uneven
    c.extend("b", 100)
    c.advance("b", 100)
    lay = _plan(c, [StepEntry(r, [1], want=[0]) for r in "abc"], decode_first=True)
    assert lay.kv_lens.tolist() == [42, 146, 38] and lay.decode_uneven  # 146 > 1.5 * mean(75.3)
    assert not _plan(c, [StepEntry("b", [1], want=[0])], decode_first=True).decode_uneven  # one row
