"""Pins the restated proAttention/proCache state machine by brute force: ring pairing,
coverage, pointer period, cache invariants (none of these retype its formulas)."""
import itertools
import random
from collections import Counter

import pytest

from oracle.state_machine import (CacheOracle, RingOracle, legal_divider_column, strides_from_dividers)


def _legal_columns(N, T, dividers=(1, 2, 4, 8)):
    divs = [d for d in dividers if d <= N]
    for mid in itertools.product(divs, repeat=T - 5):
        col = (1, 1, 1) + mid + (1, 1)  # first three and last two steps are full (redundancy_map.py:302-304)
        if legal_divider_column(col):
            yield col


def _run(N, col, use_ditango=True):
    curr, nxt = strides_from_dividers(N, col)
    ring = RingOracle(N, use_ditango=use_ditango)
    return [ring.call(t, c, n) for t, (c, n) in enumerate(zip(curr, nxt))], ring


def _aligned(N, curr, targets_before):
    """Every rank's pointer sits at its own inner offset of some block (or the step is full).
    Only then do the ranks of a ring agree on the target block; otherwise the reference
    hands chunks of other blocks round the ring and coverage is no longer exact
    (reachable after a stride-1 step, e.g. dividers ...8,4... at N=8)."""
    return curr == N or all((targets_before[x] - x) % curr == 0 for x in range(N))


@pytest.mark.parametrize("N,T", [(2, 8), (4, 9), (8, 9)])
def test_all_legal_sequences_cover_every_chunk_once(N, T):
    n_cols = 0
    n_aligned = 0
    for col in _legal_columns(N, T):
        n_cols += 1
        curr, nxt = strides_from_dividers(N, col)
        ring = RingOracle(N)
        for t in range(T):
            before = list(ring.target)
            traces = ring.call(t, curr[t], nxt[t])  # asserts send/recv pairing internally
            aligned = _aligned(N, curr[t], before)
            n_aligned += aligned
            for tr in traces:
                if aligned:
                    assert Counter(tr.out) == Counter(range(N)), (col, t, tr.rank, tr.out)
                    assert not (("local" in [k for _, k in tr.computed]) and ("own" in [k for _, k in tr.computed]))
                else:
                    # the mis-aligned case: the local chunk is merged twice by ranks whose pointer
                    # is in their own block but not on their own chunk
                    kinds = [k for _, k in tr.computed]
                    if before[tr.rank] != tr.rank and before[tr.rank] // curr[t] == tr.rank // curr[t]:
                        assert kinds[:2] == ["local", "own"] and tr.computed[0][0] == tr.computed[1][0] == tr.rank
                # the local chunk is recomputed in every call and never stored
                assert tr.rank in [c for c, _ in tr.computed]
                for slot, ids in tr.stores:
                    assert tr.rank not in ids
                # cache shape after the call
                assert tr.nblk_after == (N if nxt[t] == N else N // nxt[t])
                if nxt[t] != N:
                    assert tr.occupancy_after[tr.target_after // nxt[t]] is False
    assert n_cols >= 8 and n_aligned >= 4 * n_cols


def test_constant_stride_period_and_work():
    N = 8
    for div in (2, 4, 8):
        s = N // div
        col = (1, 1, 1) + (div,) * 12 + (1, 1)
        runs, ring = _run(N, col)
        for r in range(N):
            targets = [runs[t][r].target_after for t in range(3, 15)]
            # block pointer advances by one block per call: period N/s
            blocks = [x // s for x in targets]
            assert all((blocks[i + 1] - blocks[i]) % (N // s) == 1 % (N // s) for i in range(len(blocks) - 1))
            for t in range(4, 15):
                tr = runs[t][r]
                n_comp = len(tr.computed)
                local_in_target = any(kind == "own" for _, kind in tr.computed)
                assert n_comp == (s if local_in_target else s + 1)


def test_full_step_stores_each_chunk_separately():
    N = 4
    runs, _ = _run(N, (1, 1, 1, 4, 4, 1, 1))
    tr = runs[2][1]  # stride N with a reuse step announced
    assert sorted(slot for slot, _ in tr.stores) == [0, 2, 3]
    assert all(ids == (slot,) for slot, ids in tr.stores)


def test_two_level_ring_visits_block_once():
    """N=16: with the 8-wide inner ring every chunk of the block is still visited exactly once
    per call; exact coverage ACROSS calls only holds for the plain ring, because a full-stride
    step files the state of the i-th visited chunk under ``target + i`` (core/attention.py:208-214)
    while the two-level ring does not visit chunks in that order."""
    N = 16
    ring = RingOracle(N, use_ditango=True)
    for tr in ring.call(0, 16, 16):
        order = [c for c, _ in tr.computed]
        assert sorted(order) == list(range(N))
        r = tr.rank
        base = r // 8 * 8
        assert order[:8] == [base + (r + j) % 8 for j in range(8)]       # own small ring first
        assert order[8] == (base + 8) % 16 + (r + 7) % 8                 # inter hop keeps the position reached
    random.seed(0)
    for use_ditango in (True, False):
        for _ in range(20):
            mid = []
            prev = 1
            for _t in range(10):
                choices = [d for d in (1, 2, 4, 8) if prev == 1 or d <= prev]
                prev = random.choice(choices)
                mid.append(prev)
            col = (1, 1, 1) + tuple(mid) + (1, 1)
            curr, nxt = strides_from_dividers(N, col)
            ring = RingOracle(N, use_ditango=use_ditango)
            for t in range(len(col)):
                before = list(ring.target)
                for tr in ring.call(t, curr[t], nxt[t]):   # pairing is asserted inside
                    assert sorted(c for c, k in tr.computed if k != "local") == sorted(set(c for c, k in tr.computed if k != "local"))
                    if not use_ditango and _aligned(N, curr[t], before):
                        assert Counter(tr.out) == Counter(range(N))


def test_cache_oracle_rules():
    c = CacheOracle(8)
    for i in range(8):
        c.store_block(i, (i,))
    c.update_cache_blocks(2, 1)  # 8 -> 4 blocks, block 1 invalidated
    assert c.curr_block_num == 4 and c.slots == [(0, 1), None, (4, 5), (6, 7)]
    c.update_cache_blocks(4, 0)  # 4 -> 2 blocks; empty members are skipped
    assert c.slots == [None, (4, 5, 6, 7)]
    with pytest.raises(AssertionError):
        c.update_cache_blocks(2, 0)  # refining (more blocks) is illegal (cache.py:65)
    c.update_cache_blocks(8, 0)
    assert c.slots == [None] * 8 and c.curr_block_num == 8
    c.update_cache_blocks(0, 0)
    assert c.slots == [None] and c.curr_block_num == 1
    with pytest.raises(IndexError):
        c.get_block(3)


def test_memory_guard_forces_full_refresh():
    N = 4
    ring = RingOracle(N, memory_ok=lambda cache, nxt: False)
    curr, nxt = strides_from_dividers(N, (1, 1, 1, 2, 2, 1, 1))
    tr = ring.call(2, curr[2], nxt[2])[0]
    assert tr.next_stride == N and tr.stores == [] and tr.nblk_after == N
