"""Oracle and product against the committed schedule fixtures (tests/golden/*.npz, written by
tests/golden/make_schedule_fixtures.py from the oracle): bit-exact."""
import importlib.util
import os

import numpy as np
import pytest
import torch


GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
_spec = importlib.util.spec_from_file_location("make_schedule_fixtures", os.path.join(GOLDEN, "make_schedule_fixtures.py"))
gen = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(gen)

STRIDE = np.load(os.path.join(GOLDEN, "stride_schedules.npz"))
MASKS = np.load(os.path.join(GOLDEN, "mask_schedules.npz"))
N = 8


@pytest.mark.parametrize("name", list(gen.MAPS))
def test_oracle_reproduces_stride_fixture(name):
    fresh = gen.stride_schedule(name)
    for key, val in fresh.items():
        assert np.array_equal(val, STRIDE[key]), key


@pytest.mark.parametrize("name", list(gen.MASKS))
def test_oracle_reproduces_mask_fixture(name):
    fresh = gen.mask_schedule(name)
    for key, val in fresh.items():
        assert np.array_equal(val, MASKS[key]), key
    T, L, C, p, seed, diag = gen.MASKS[name]
    cnt = MASKS[f"{name}/counts"]
    assert (cnt.sum(-1) == C).all()                       # every chunk is computed or reused
    assert (cnt[0, :, 0] == C).all()                      # cold first step
    if T > 1 and 0 < p < 1:
        realised = MASKS[f"{name}/mask"][1:].mean() * (C / (C - 1) if diag >= 0 else 1.0)
        assert abs(realised - p) < 0.02


@pytest.mark.parametrize("name", list(gen.MAPS))
@pytest.mark.parametrize("rank", [0, 3, 7])
def test_product_plan_reproduces_stride_fixture(name, rank):
    """The host-side planner of proAttention (no GPU needed in dry-run mode) on the shipped maps."""
    from ditango_amd.core import config, parallel_state, redundancy_map as rmod
    from ditango_amd.core.attention import proAttention
    from ditango_amd.utils import update_timestep
    fn, pct, dv = gen.MAPS[name]
    div = STRIDE[f"{name}/dividers"]
    T, L = div.shape
    parallel_state.init_local_groups(N, rank)
    cfg = config.init_config(None, num_inference_steps=T, num_layers=L, stride_percentiles=pct, stride_dividers=dv)
    rmod.destroy_redundancy_map()
    try:
        rm = rmod.init_redundancy_map(cfg, redun_map_path=os.path.join(GOLDEN, fn), quiet=True)
        assert np.array_equal(rm.divider_map.numpy(), div)
        group = parallel_state.get_usp_group()
        layers = [proAttention(l, group, dry_run=True) for l in range(0, L, 7)]
        for t in range(T):
            update_timestep(t)
            for attn in layers:
                l = attn.layer_id
                attn.attn(None, None, None)
                p = attn.last_plan
                ids = [c for c, _ in p.computed]
                want = STRIDE[f"{name}/computed"][rank, l, t]
                assert ids == [int(c) for c in want[want >= 0]], (name, rank, l, t)
                wm = STRIDE[f"{name}/merged"][rank, l, t]
                assert p.reuse_merged == [int(c) for c in wm[wm >= 0]], (name, rank, l, t)
                assert p.target_after == STRIDE[f"{name}/target_after"][rank, l, t]
                assert p.nblk_after == STRIDE[f"{name}/nblk_after"][rank, l, t]
    finally:
        rmod.destroy_redundancy_map()
        parallel_state.destroy_local_groups()
        update_timestep(0)


def test_product_draws_the_fixture_masks():
    from ditango_amd.core.redundancy_map import make_bernoulli_mask
    for name, (T, L, C, p, seed, diag) in gen.MASKS.items():
        assert np.array_equal(make_bernoulli_mask(T, L, C, p, seed=seed, diag=diag), MASKS[f"{name}/mask"]), name


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(gen.MASKS))
def test_device_schedule_builder_reproduces_mask_fixture(hip, name):
    T, L, C, p, seed, diag = gen.MASKS[name]
    comp, reu, cnt = hip.build_schedule_table(torch.from_numpy(MASKS[f"{name}/mask"]).cuda(), diag)
    torch.cuda.synchronize()
    assert np.array_equal(comp.cpu().numpy(), MASKS[f"{name}/compute_ids"])
    assert np.array_equal(reu.cpu().numpy(), MASKS[f"{name}/reuse_ids"])
    assert np.array_equal(cnt.cpu().numpy(), MASKS[f"{name}/counts"])
