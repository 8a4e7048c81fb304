"""Divider-map generation and refinement on the three redundancy maps the reference ships
(``configs/*/redundancy_map_50_*.pt`` and the percentiles/dividers of ``configs/*/config.yaml``,
copied as data under tests/golden/)."""
import os
from collections import Counter

import numpy as np
import pytest
import torch

from oracle import divider_map as od
from oracle.state_machine import RingOracle, legal_divider_column, strides_from_dividers

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
# (file, layers, stride-percentiles of the model's config.yaml, dividers)
MODELS = {
    "cogvideox-5b": ("redundancy_map_50_42.pt", 42, [0, 40, 90], [8, 4, 2, 1]),
    "hunyuanvideo": ("redundancy_map_50_60.pt", 60, [0, 40, 90], [8, 4, 2, 1]),
    "stepvideo": ("redundancy_map_50_48.pt", 48, [0, 0, 90], [8, 4, 2, 1]),
}
# Divider histograms and double-count tallies that an independent restatement of the same
# reference functions, written earlier and separately from this oracle, produced for N=8; agreement of two
# independent restatements, not reference output.
INDEPENDENT_HIST = {
    "cogvideox-5b": {1: 381, 2: 946, 4: 773},
    "hunyuanvideo": {1: 560, 2: 1379, 4: 1061},
    "stepvideo": {1: 472, 2: 1928},
}
INDEPENDENT_DOUBLE_COUNT = {"cogvideox-5b": 280, "hunyuanvideo": 356, "stepvideo": 0}
INDEPENDENT_MEAN_COMPUTED = {"cogvideox-5b": 4.49, "hunyuanvideo": 4.53, "stepvideo": 5.18}


def _load(name):
    fn, L, pct, dv = MODELS[name]
    red = torch.load(os.path.join(GOLDEN, fn), map_location="cpu", weights_only=True)
    assert red.dtype == torch.float32 and tuple(red.shape) == (50, L)
    return red, pct, dv


@pytest.mark.parametrize("name", list(MODELS))
def test_fixture_properties(name):
    red, _, _ = _load(name)
    assert (red[0] == 0).all()          # the first step has no predecessor to compare with
    assert (red[1:] > 0).all() and torch.isfinite(red).all()


@pytest.mark.parametrize("name", list(MODELS))
def test_generated_map_rules_and_histogram(name):
    red, pct, dv = _load(name)
    div, percentiles = od.generate_divider_map(red.numpy(), 8, pct, dv)
    T, L = div.shape
    # rules the source states, checked on the result rather than re-derived:
    assert (div[T - 1] == 1).all()                       # last step full
    assert (div[0] == 1).all()                           # zero redundancy keeps the initial 1
    assert set(np.unique(div)) <= set(dv)
    nz = red.numpy()[red.numpy() > 0].astype(np.float64)
    # bins are monotone in the redundancy: a larger value never gets a larger divider
    body = div[1:T - 1].ravel()
    vals = red.numpy()[1:T - 1].ravel()
    order = np.argsort(vals, kind="stable")
    assert (np.diff(body[order]) <= 0).all()
    # the share of the top bin follows the top percentile (90 -> about a tenth gets divider 1)
    top = np.mean(body == dv[3])
    assert abs(top - (100 - pct[2]) / 100) < 0.01
    refined, changes = od.refine_divider_map(div)
    assert dict(Counter(int(x) for x in refined.ravel())) == INDEPENDENT_HIST[name]
    # refined map: legal transitions in every layer, first three and last two steps full
    for l in range(L):
        assert legal_divider_column(refined[:, l])
    assert (refined[:3] == 1).all() and (refined[T - 2:] == 1).all()
    # refinement only ever lowers a divider to 1
    assert ((refined == div) | (refined == 1)).all()
    assert changes == int((refined != div).sum())


@pytest.mark.parametrize("name", list(MODELS))
def test_schedule_statistics_agree_with_independent_restatement(name):
    """Run the ring oracle over the whole refined map (8 ranks x L layers x 50 steps)."""
    red, pct, dv = _load(name)
    div, _ = od.generate_divider_map(red.numpy(), 8, pct, dv)
    refined, _ = od.refine_divider_map(div)
    N = 8
    T, L = refined.shape
    double = 0
    computed = 0
    calls = 0
    for l in range(L):
        curr, nxt = strides_from_dividers(N, refined[:, l])
        ring = RingOracle(N, layer_id=l)
        for t in range(T):
            for tr in ring.call(t, curr[t], nxt[t]):
                kinds = [k for _, k in tr.computed]
                double += ("local" in kinds and "own" in kinds)
                computed += len(tr.computed)
                calls += 1
    assert calls == N * L * T
    assert double == INDEPENDENT_DOUBLE_COUNT[name]
    assert abs(computed / calls - INDEPENDENT_MEAN_COMPUTED[name]) < 0.006


@pytest.mark.parametrize("name", list(MODELS))
def test_product_redundancy_map_equals_oracle(name, tmp_path):
    from ditango_amd.core import config, parallel_state, redundancy_map as rmod
    red, pct, dv = _load(name)
    fn, L, _, _ = MODELS[name]
    parallel_state.init_local_groups(8, 0)
    cfg = config.init_config(None, num_inference_steps=50, num_layers=L, stride_percentiles=pct, stride_dividers=dv,
                             ditango_base=str(tmp_path), model_name=name)
    rmod.destroy_redundancy_map()
    try:
        rm = rmod.init_redundancy_map(cfg, redun_map_path=os.path.join(GOLDEN, fn), quiet=True)
        div, _ = od.generate_divider_map(red.numpy(), 8, pct, dv)
        refined, _ = od.refine_divider_map(div)
        assert rm.divider_map.dtype == torch.long
        assert np.array_equal(rm.divider_map.numpy(), refined)
        for t in (0, 3, 17, 48, 49):
            for l in (0, L // 2, L - 1):
                assert rm.get_curr_isp_stride(t, l) == od.curr_stride(refined, 8, t, l)
                assert rm.get_next_isp_stride(t, l) == od.next_stride(refined, 8, t, l)
        # save / reload round trip in the reference's file format (a bare fp32 tensor)
        path = rmod.save_redundancy_map(path=str(tmp_path / "m.pt"), override=True)
        back = torch.load(path, weights_only=True)
        assert torch.equal(back, red)
        assert rmod.save_divider_map(path=str(tmp_path / "d.pt")) is not None
        assert torch.equal(torch.load(str(tmp_path / "d.pt"), weights_only=True), rm.divider_map)
    finally:
        rmod.destroy_redundancy_map()
        parallel_state.destroy_local_groups()


def test_divider_generation_edge_cases():
    red = np.zeros((6, 2), dtype=np.float32)
    div, pct = od.generate_divider_map(red, 8)
    assert pct is None and (div == 1).all()                       # nothing positive: map untouched
    red[1:5] = np.arange(8, dtype=np.float32).reshape(4, 2) + 1
    div, pct = od.generate_divider_map(red, 8, [25, 50, 75], [8, 4, 2, 1])
    assert div[1].tolist() == [8, 8] and div[4].tolist() == [1, 1] and div[5].tolist() == [1, 1]
    # base weight smaller than the divider clamps to the base weight (redundancy_map.py:262-263)
    div4, _ = od.generate_divider_map(red, 4, [25, 50, 75], [8, 4, 2, 1])
    assert div4[1].tolist() == [4, 4]
    # base weight not divisible: falls to the smallest listed divider that divides it (:264-271)
    div6, _ = od.generate_divider_map(red, 6, [25, 50, 75], [8, 4, 2, 1])
    assert set(np.unique(div6)) <= {1, 2, 6}


# ---- against the reference's own output ---------------------------------------------------------
# tests/golden/divider_maps.npz holds what the reference's generate_divider_map_from_redundancy +
# _refine_divider_map (core/redundancy_map.py:199-326) return on the shipped maps for ring sizes
# 2, 4, 8 and 16 (written by tests/golden/make_divider_fixtures.py, which imports those two
# functions from the reference tree).  Integer work: bit exact.
REFERENCE_OUTPUT = np.load(os.path.join(GOLDEN, "divider_maps.npz"))


@pytest.mark.parametrize("N", [2, 4, 8, 16])
@pytest.mark.parametrize("name", list(MODELS))
def test_oracle_equals_reference_output(name, N):
    red, pct, dv = _load(name)
    key = name.replace("-", "_")
    assert np.array_equal(REFERENCE_OUTPUT[f"{key}.redundancy"], red.numpy())          # same inputs
    assert list(REFERENCE_OUTPUT[f"{key}.percentiles"]) == pct and list(REFERENCE_OUTPUT[f"{key}.dividers"]) == dv
    div, thresholds = od.generate_divider_map(red.numpy(), N, pct, dv)
    assert np.array_equal(np.asarray(thresholds, dtype=np.float64), REFERENCE_OUTPUT[f"{key}.N{N}.thresholds"])
    assert np.array_equal(div, REFERENCE_OUTPUT[f"{key}.N{N}.generated"])
    refined, changes = od.refine_divider_map(div)
    assert np.array_equal(refined, REFERENCE_OUTPUT[f"{key}.N{N}.refined"])
    assert changes == int(REFERENCE_OUTPUT[f"{key}.N{N}.changes"])


@pytest.mark.parametrize("N", [2, 4, 8, 16])
@pytest.mark.parametrize("name", list(MODELS))
def test_product_equals_reference_output(name, N):
    """The host-side RedundancyMap of the package (what init_redundancy_map builds from a .pt file)."""
    from ditango_amd.core import config, parallel_state, redundancy_map as rmod

    red, pct, dv = _load(name)
    key = name.replace("-", "_")
    parallel_state.init_local_groups(N, 0)
    cfg = config.init_config(None, num_inference_steps=50, num_layers=MODELS[name][1], stride_percentiles=pct,
                             stride_dividers=dv)
    rmod.destroy_redundancy_map()
    try:
        rm = rmod.RedundancyMap(cfg)
        rm.redundancy_map = red
        rm.generate_divider_map_from_redundancy(custom_percentages=pct, custom_dividers=dv)
        assert np.array_equal(rm.divider_map.numpy(), REFERENCE_OUTPUT[f"{key}.N{N}.generated"])
        rm._refine_divider_map()
        assert np.array_equal(rm.divider_map.numpy(), REFERENCE_OUTPUT[f"{key}.N{N}.refined"])
    finally:
        rmod.destroy_redundancy_map()
        parallel_state.destroy_local_groups()


def test_golden_stride_schedules_start_from_the_reference_dividers():
    """The committed stride schedules (made from the oracle) were generated from dividers that equal
    the reference's own refined maps for a ring of 8."""
    stride = np.load(os.path.join(GOLDEN, "stride_schedules.npz"))
    for short, key in (("cogvideox", "cogvideox_5b"), ("hunyuanvideo", "hunyuanvideo"), ("stepvideo", "stepvideo")):
        assert np.array_equal(stride[f"{short}/dividers"], REFERENCE_OUTPUT[f"{key}.N8.refined"])
