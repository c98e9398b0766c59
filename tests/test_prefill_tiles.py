"""The host-side list of query tiles for the prefill attention kernel: a partition of the new
tokens, ordered so that the launch is balanced."""

import random

from torchllms_amd.kernels.ops import (
    PREFILL_SPLIT_BLOCKS,
    prefill_key_groups,
    prefill_tile_count,
    prefill_tiles,
)


def _cost(row, q0, qo, kv, qpt, window):
    q_len = qo[row + 1] - qo[row]
    pos0 = kv[row] - q_len
    hi = pos0 + min(q0 + qpt, q_len) - 1
    lo = max(pos0 + q0 - window + 1, 0) if window > 0 else 0
    return hi - lo + 1


def test_tiles_are_a_partition_whatever_the_order():
    rng = random.Random(0)
    for _ in range(50):
        n_rows = rng.randint(1, 5)
        first = rng.randint(0, n_rows - 1)
        q_lens = [rng.randint(1, 300) for _ in range(n_rows)]
        kv = [q + rng.randint(0, 500) for q in q_lens]
        qo = [0]
        for q in q_lens:
            qo.append(qo[-1] + q)
        qpt = rng.choice([8, 16, 32, 128])
        window = rng.choice([0, 0, 7, 100])
        rows, q0s = prefill_tiles(qo, first, n_rows, qpt, kv, window)
        want = sorted((r, q0) for r in range(first, n_rows) for q0 in range(0, q_lens[r], qpt))
        assert sorted(zip(rows, q0s)) == want
        assert prefill_tile_count(qo, first, n_rows, qpt) == len(want)
        plain_rows, plain_q0s = prefill_tiles(qo, first, n_rows, qpt)  # without lengths: in natural order
        assert list(zip(plain_rows, plain_q0s)) == want


def test_a_launch_starts_its_longest_tiles_first():
    qo, kv, qpt = [0, 100, 8292], [5000, 8192], 32
    rows, q0s = prefill_tiles(qo, 0, 2, qpt, kv, 0)
    costs = [_cost(r, q, qo, kv, qpt, 0) for r, q in zip(rows, q0s)]
    assert costs == sorted(costs, reverse=True)
    assert rows[0] == 1 and rows[-1] == 1 and 0 in rows  # the short row's tiles lie where their length puts them


def test_two_sets_of_waves_for_launches_that_fit_at_once_and_then_longest_first():
    qo, kv, qpt, heads = [0, 2048], [2048], 32, 8
    n = prefill_tile_count(qo, 0, 1, qpt)
    assert n * heads <= PREFILL_SPLIT_BLOCKS and prefill_key_groups(n, heads, 2048) == 2
    assert prefill_key_groups(n, heads, 2048 + 4096) == 1  # behind a long prefix two blocks a CU do better
    assert prefill_key_groups(n // 2, heads, 2048 + 8192) == 2  # too few blocks to give every CU two
    rows, q0s = prefill_tiles(qo, 0, 1, qpt, kv, 0)
    costs = [_cost(r, q, qo, kv, qpt, 0) for r, q in zip(rows, q0s)]
    assert costs == sorted(costs, reverse=True)
    assert prefill_key_groups(prefill_tile_count([0, 8192], 0, 1, qpt), heads) == 1
    assert prefill_key_groups(PREFILL_SPLIT_BLOCKS // heads + 1, heads) == 1
