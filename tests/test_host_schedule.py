"""The product's host-side schedule (closed-form ring delivery, pointer, cache
bookkeeping) must equal the lock-step ring simulation of the oracle bit for bit."""
import random

import pytest
import torch

from oracle.state_machine import RingOracle, legal_divider_column, strides_from_dividers


@pytest.fixture
def ditango_env():
    from ditango_amd.core import config, parallel_state, redundancy_map
    from ditango_amd import utils

    def make(N, rank, T, L, use_ditango=True):
        parallel_state.init_local_groups(N, rank)
        config.init_config(None, num_inference_steps=T, num_layers=L, use_ditango=use_ditango)
        redundancy_map.destroy_redundancy_map()
        redundancy_map._redundancy_map = redundancy_map.RedundancyMap(config.get_config())
        return redundancy_map.get_redundancy_map()

    yield make
    from ditango_amd.core import parallel_state as ps, redundancy_map as rmod
    rmod.destroy_redundancy_map()
    ps.destroy_local_groups()
    utils.update_timestep(0)


def _random_column(T, N, rng):
    mid, prev = [], 1
    for _ in range(T - 5):
        prev = rng.choice([d for d in (1, 2, 4, 8) if d <= N and (prev == 1 or d <= prev)])
        mid.append(prev)
    col = (1, 1, 1) + tuple(mid) + (1, 1)
    assert legal_divider_column(col)
    return col


@pytest.mark.parametrize("N,use_ditango", [(2, True), (4, True), (8, True), (16, True), (16, False)])
def test_plan_matches_ring_oracle(ditango_env, N, use_ditango):
    from ditango_amd.core.attention import proAttention
    from ditango_amd.core.parallel_state import get_usp_group
    from ditango_amd.utils import update_timestep

    T = 14
    rng = random.Random(N)
    for trial in range(6):
        col = _random_column(T, N, rng)
        curr, nxt = strides_from_dividers(N, col)
        ring = RingOracle(N, use_ditango=use_ditango)
        oracle_traces = [ring.call(t, curr[t], nxt[t]) for t in range(T)]
        for rank in range(N):
            rm = ditango_env(N, rank, T, 1, use_ditango)
            rm.divider_map[:, 0] = torch.tensor(col)
            attn = proAttention(0, get_usp_group(), dry_run=True)
            for t in range(T):
                update_timestep(t)
                attn.attn(None, None, None)
                p, o = attn.last_plan, oracle_traces[t][rank]
                ctx = (col, rank, t)
                assert (p.curr_stride, p.next_stride) == (o.curr_stride, o.next_stride), ctx
                assert p.reuse_probed == o.reuse_probed, ctx
                assert p.reuse_merged == o.reuse_merged, ctx
                assert p.computed == o.computed, ctx
                assert p.stores == o.stores, ctx
                assert p.flushes == o.flushes, ctx
                assert p.target_after == o.target_after, ctx
                assert p.nblk_after == o.nblk_after, ctx
                assert p.occupancy_after == o.occupancy_after, ctx


def test_strides_follow_divider_map(ditango_env):
    from oracle import divider_map as od
    rm = ditango_env(8, 0, 6, 3)
    rm.divider_map = torch.tensor([[1, 1, 1], [8, 4, 2], [8, 2, 1], [4, 2, 1], [1, 1, 1], [2, 2, 2]])
    div = rm.divider_map.numpy()
    for t in range(6):
        for l in range(3):
            assert rm.get_curr_isp_stride(t, l) == od.curr_stride(div, 8, t, l)
            assert rm.get_next_isp_stride(t, l) == od.next_stride(div, 8, t, l)
    assert rm.get_next_isp_stride(5, 0) == 8  # last step announces a full refresh
    # the cache's accessor of the same name reads the current step
    from ditango_amd.core.cache import proCache
    from ditango_amd.utils import update_timestep
    update_timestep(2)
    assert proCache(8, 1).get_curr_isp_stride(1) == od.curr_stride(div, 8, 2, 1)
    update_timestep(0)
    rm.auto_setting = True
    assert rm.get_curr_isp_stride(1, 0) == 8 and rm.get_next_isp_stride(1, 0) == 8
    rm.auto_setting = False
    # base weight smaller than the divider -> stride 1 (redundancy_map.py:63-64)
    rm.base_weight = 4
    assert rm.get_curr_isp_stride(1, 0) == 1


def test_set_pattern_rows(ditango_env):
    rm = ditango_env(8, 0, 5, 6)
    rm.set_pattern_for_rows(range(1, 3), [2, 4], [8, 4, 2])
    assert rm.divider_map[1].tolist() == [8, 8, 4, 4, 2, 2] and rm.divider_map[0].tolist() == [1] * 6
    rm.set_full_stride_for_rows([3])
    assert rm.divider_map[3].tolist() == [8] * 6
    with pytest.raises(ValueError):
        rm.set_pattern_for_row(9, [], [1])
    rm.reset_map()
    assert int(rm.divider_map.sum()) == 30


def test_memory_guard_falls_back_to_full_refresh(ditango_env):
    """An over-budget prediction turns the announced stride into N (core/attention.py:97-98)."""
    from ditango_amd.core.cache import proCache
    c = proCache(8, 0)
    c.block_size_mb = 100.0
    c.memory_constraint = 1000.0
    c.memory_probe = lambda: 500.0
    assert c.pass_memory_check(8, 0) is True          # full refresh is always fine
    assert c.pass_memory_check(2, 0) is True           # 4 blocks * 100 MB + 500 <= 1000
    assert c.pass_memory_check(1, 0) is False          # 8 blocks * 100 MB + 500 > 1000
    c.out_block_cache = [object()] * 8                 # already holding as many blocks as predicted
    assert c.pass_memory_check(1, 0) is True


@pytest.mark.parametrize("N,col,trip", [
    (8, (1, 1, 1, 4, 4, 2, 2, 1, 1), {2}),          # guard trips on the step that announces stride 2
    (8, (1, 1, 1, 4, 4, 2, 2, 1, 1), {2, 3}),       # ... and again on the next one
    (8, (1, 1, 1, 8, 8, 4, 2, 2, 1, 1), {2}),       # stride 1 announced: 8 blocks predicted, none held
    (8, (1, 1, 1, 2, 2, 2, 2, 2, 1, 1), {4}),       # mid-run: one of two blocks held, the other predicted
    (4, (1, 1, 1, 2, 2, 2, 4, 4, 1, 1), {2, 5}),
    (16, (1, 1, 1, 8, 8, 4, 4, 2, 1, 1), {2, 6}),   # two-level ring
])
def test_plan_with_a_tripping_memory_guard_matches_ring_oracle(ditango_env, N, col, trip):
    """The stride-mode fallback (core/attention.py:97-98 with core/cache.py:103-128): when the predicted
    allocation exceeds the budget, only this call's announced stride becomes N -- nothing is stored, the
    cache is reset to N empty slots -- and the next call reads its stride from the map again, so it probes
    block ids of an empty cache and those chunks drop out of the softmax.  The planner, fed the same three
    quantities as the restated guard, must follow the lock-step ring step for step."""
    from ditango_amd.core.attention import proAttention
    from ditango_amd.core.parallel_state import get_usp_group
    from ditango_amd.utils import update_timestep

    T = len(col)
    curr, nxt = strides_from_dividers(N, col)
    now = {"t": 0}
    probe = lambda: 950.0 if now["t"] in trip else 0.0      # MB allocated; budget 1000, a block is 100
    ring = RingOracle(N, memory_probe=probe, block_size_mb=100.0, memory_constraint=1000.0)
    oracle_traces = []
    for t in range(T):
        now["t"] = t
        oracle_traces.append(ring.call(t, curr[t], nxt[t]))
    tripped = {t for t in range(T) if oracle_traces[t][0].next_stride != nxt[t]}
    assert tripped, "the case is meant to trip the guard"
    dropped = 0
    for rank in range(N):
        rm = ditango_env(N, rank, T, 1)
        rm.divider_map[:, 0] = torch.tensor(col)
        attn = proAttention(0, get_usp_group(), dry_run=True)
        attn.cache.block_size_mb, attn.cache.memory_constraint, attn.cache.memory_probe = 100.0, 1000.0, probe
        for t in range(T):
            now["t"] = t
            update_timestep(t)
            attn.attn(None, None, None)
            p, o = attn.last_plan, oracle_traces[t][rank]
            ctx = (col, rank, t)
            assert (p.curr_stride, p.next_stride) == (o.curr_stride, o.next_stride), ctx
            assert p.reuse_probed == o.reuse_probed and p.reuse_merged == o.reuse_merged, ctx
            assert p.computed == o.computed and p.stores == o.stores and p.flushes == o.flushes, ctx
            assert (p.target_after, p.nblk_after, p.occupancy_after) == (o.target_after, o.nblk_after, o.occupancy_after), ctx
            if t in tripped:
                assert p.next_stride == N and p.stores == [] and p.nblk_after == N and not any(p.occupancy_after), ctx
            if t - 1 in tripped and curr[t] != N:
                # the desync: blocks are probed, none is there, fewer than N chunks reach the softmax
                assert p.reuse_probed and p.reuse_merged == [], ctx
                dropped += N - len({c for c, _ in p.computed})
    assert dropped > 0


def test_mask_mode_arena_consults_the_memory_guard(ditango_env):
    """ensure_arena uses the probe and budget of pass_memory_check (core/cache.py:103-128): an arena
    that would push the allocation over the budget is refused (once, with a warning), a fitting one is
    allocated; release() forgets the refusal."""
    from ditango_amd.core.cache import proCache
    c = proCache(8, 0)
    need_mb = 9 * 1 * 64 * 2 * (2 * 64 + 4) / 2 ** 20          # 8 chunks + the local state
    c.memory_constraint = 100.0
    c.memory_probe = lambda: 100.0 - need_mb / 2
    assert c.ensure_arena(8, 1, 64, 2, 64, torch.device("cpu")) is False
    assert c.arena_out is None and c.arena_refused == (8, 1, 64, 2, 64)
    c.memory_probe = lambda: 0.0
    assert c.ensure_arena(8, 1, 64, 2, 64, torch.device("cpu")) is False       # a refusal sticks for that shape
    c.release()
    assert c.ensure_arena(8, 1, 64, 2, 64, torch.device("cpu")) is True
    assert tuple(c.arena_out.shape) == (8, 1, 64, 2, 64) and tuple(c.arena_lse.shape) == (8, 1, 2, 64)
    assert c.arena_valid == [False] * 8
    c.clear()                                                                   # the reference's clear() keeps the states
    assert c.arena_out is not None


def test_lse_layout_when_query_and_head_counts_coincide():
    """With Sq == H the shape cannot tell [B,H,S] from [B,S,H]: a 4-D [.,.,.,1] tensor is the running layout of
    utils.py:49 ([B,S,H,1]), a 3-D one flash-attn's [B,H,S]; everywhere else shape and strides decide."""
    import torch
    from ditango_amd._hip import DT_LSE_BHS, DT_LSE_BSH, DitangoHipError, lse_layout_of
    assert lse_layout_of(torch.zeros(2, 5, 5, 1), 2, 5, 5) == DT_LSE_BSH
    assert lse_layout_of(torch.zeros(2, 5, 5), 2, 5, 5) == DT_LSE_BHS
    assert lse_layout_of(torch.zeros(1, 5, 7, 1), 1, 5, 7) == DT_LSE_BSH
    assert lse_layout_of(torch.zeros(1, 7, 5), 1, 5, 7) == DT_LSE_BHS
    assert lse_layout_of(torch.zeros(1, 7, 5).transpose(1, 2), 1, 5, 7) == DT_LSE_BHS      # a view of [B,H,S] storage
    assert lse_layout_of(torch.zeros(1, 5, 7).transpose(1, 2), 1, 5, 7) == DT_LSE_BSH
    with pytest.raises(DitangoHipError):
        lse_layout_of(torch.zeros(1, 6, 7), 1, 5, 7)
