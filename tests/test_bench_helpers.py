"""Host-side pieces of bench.py that decide WHAT is timed: the stratified visiting order of the
schedule rows (so that the headline does not move with --steps) and the profile lookup."""
import importlib.util
import json
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_every_prefix_of_the_stratified_order_has_the_schedules_mix():
    bench = _bench()
    from ditango_amd.core.redundancy_map import make_bernoulli_mask
    T, L, C, p = 50, 60, 8, 0.6
    mask = make_bernoulli_mask(T, L, C, p, seed=0, diag=0)
    counts = [int(C - mask[t, l].sum()) for t in range(1, T) for l in range(L)]      # chunks recomputed per row
    order = bench.stratified_order(counts)
    assert sorted(order) == list(range(len(counts)))                                 # a permutation: every row once
    population = float(np.mean(counts))
    for k, tol in ((10, 0.06), (20, 0.04), (40, 0.01), (120, 0.01), (500, 0.01)):
        mean_k = float(np.mean([counts[i] for i in order[:k]]))
        assert abs(mean_k - population) <= tol * population, (k, mean_k, population)
        # ... and every count of the schedule is represented in proportion (to within one row)
        if k >= 40:
            for c in set(counts):
                share = counts.count(c) / len(counts) * k
                assert abs(sum(1 for i in order[:k] if counts[i] == c) - share) <= 1.0, (k, c)
    # the plain prefix of the schedule, which an unstratified benchmark would time, is off by several percent at 20 steps
    assert abs(float(np.mean(counts[:20])) - population) > 0.04 * population
    assert bench.stratified_order([5]) == [0] and sorted(bench.stratified_order([3, 3, 3])) == [0, 1, 2]


def test_traffic_profiles_are_keyed_by_launch_shape():
    bench = _bench()
    for wl, typical in (("hunyuanvideo", "4"), ("cogvideox", "5"), ("sweep", "16")):
        t = bench.load_traffic(wl)
        assert isinstance(t.get("attn_fwd"), dict) and typical in t["attn_fwd"], wl
        assert all(int(v) > 0 for v in t["attn_fwd"].values())
        assert isinstance(t.get("merge_states"), dict) and len(t["merge_states"]) == 1
    assert bench.load_traffic("no-such-workload") == {}


def test_rotation_cycles_through_its_argument_sets():
    bench = _bench()
    seen = []
    r = bench.Rotation(seen.append, 3)
    for _ in range(7):
        r()
    assert seen == [0, 1, 2, 0, 1, 2, 0]


def test_power_readings_come_from_the_hwmon_files_in_watts(tmp_path, monkeypatch):
    """bench.py reads the package power and its cap from the GPU's hwmon node (microwatts); a box without the
    files yields None, never an exception."""
    bench = _bench()
    import glob as glob_module
    node = tmp_path / "card0" / "device" / "hwmon" / "hwmon3"
    node.mkdir(parents=True)
    (node / "power1_input").write_text("1357000000\n")
    (node / "power1_cap").write_text("1400000000\n")
    real_glob = glob_module.glob
    monkeypatch.setattr(glob_module, "glob", lambda pat: real_glob(pat.replace("/sys/class/drm", str(tmp_path))))
    assert bench._hwmon_watts("input") == 1357.0 and bench.power_cap_w() == 1400.0
    assert bench._hwmon_watts("average") is None
    (node / "power1_input").write_text("not a number\n")
    assert bench._hwmon_watts("input") is None
