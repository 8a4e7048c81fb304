#!/usr/bin/env python3
"""Writes the schedule fixtures next to this file (run from the repository root:
``python tests/golden/make_schedule_fixtures.py``).

These vectors come from the CPU oracle, not from the reference (which ships no tests and was
never run): they freeze the schedules the oracle derives today, so that a later change to the
oracle OR to the product shows up as a difference against committed data.

* ``stride_schedules.npz``  for each redundancy map the reference ships (tests/golden/*.pt, with
  the percentiles / dividers of its config.yaml) and every ring rank of 8: the refined divider
  map and, per (layer, step), the chunk ids the rank computes in launch order (-1 padded), the
  block ids it merges from the cache, the target pointer and the number of cache blocks after
  the call.
* ``mask_schedules.npz``    for the seeded reuse masks of the BASELINE configurations 2-5: the
  mask and the compute / reuse id lists and counts of every (step, layer).
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import divider_map as od  # noqa: E402
from oracle import mask_schedule as ms  # noqa: E402
from oracle.state_machine import RingOracle, strides_from_dividers  # noqa: E402

MAPS = {  # name: (file, percentiles, dividers)  -- configs/<model>/config.yaml of the reference
    "cogvideox": ("redundancy_map_50_42.pt", [0, 40, 90], [8, 4, 2, 1]),
    "stepvideo": ("redundancy_map_50_48.pt", [0, 0, 90], [8, 4, 2, 1]),
    "hunyuanvideo": ("redundancy_map_50_60.pt", [0, 40, 90], [8, 4, 2, 1]),
}
MASKS = {  # name: (T, L, C, reuse probability, seed, diag)
    "cogvideox": (50, 42, 8, 0.5, 0, 0),
    "hunyuanvideo": (50, 60, 8, 0.6, 0, 0),
    "stepvideo": (50, 48, 8, 0.75, 0, 0),
    "sweep_0.0": (2, 60, 32, 0.0, 0, -1),   # step 0 fills the cache, step 1 is the measured one
    "sweep_0.25": (2, 60, 32, 0.25, 0, -1),
    "sweep_0.5": (2, 60, 32, 0.5, 0, -1),
    "sweep_0.75": (2, 60, 32, 0.75, 0, -1),
    "sweep_0.9": (2, 60, 32, 0.9, 0, -1),
}
N = 8
MAX_COMPUTED = N + 1  # a call computes at most the local chunk plus a full block


def stride_schedule(name):
    fn, pct, dv = MAPS[name]
    red = torch.load(os.path.join(HERE, fn), weights_only=True).numpy()
    div, _ = od.generate_divider_map(red, N, pct, dv)
    refined, _ = od.refine_divider_map(div)
    T, L = refined.shape
    computed = np.full((N, L, T, MAX_COMPUTED), -1, dtype=np.int8)
    merged = np.full((N, L, T, N), -1, dtype=np.int8)
    target = np.zeros((N, L, T), dtype=np.int8)
    nblk = np.zeros((N, L, T), dtype=np.int8)
    for l in range(L):
        curr, nxt = strides_from_dividers(N, refined[:, l])
        ring = RingOracle(N, layer_id=l)
        for t in range(T):
            for tr in ring.call(t, curr[t], nxt[t]):
                ids = [c for c, _ in tr.computed]
                computed[tr.rank, l, t, :len(ids)] = ids
                merged[tr.rank, l, t, :len(tr.reuse_merged)] = tr.reuse_merged
                target[tr.rank, l, t] = tr.target_after
                nblk[tr.rank, l, t] = tr.nblk_after
    return {f"{name}/dividers": refined.astype(np.int8), f"{name}/computed": computed, f"{name}/merged": merged,
            f"{name}/target_after": target, f"{name}/nblk_after": nblk}


def mask_schedule(name):
    T, L, C, p, seed, diag = MASKS[name]
    mask = ms.seeded_mask(T, L, C, p, seed=seed, diag=diag)
    comp, reu, cnt = ms.build_schedule_table(mask, diag)
    return {f"{name}/mask": mask.astype(np.uint8), f"{name}/compute_ids": comp.astype(np.int8),
            f"{name}/reuse_ids": reu.astype(np.int8), f"{name}/counts": cnt.astype(np.int8)}


def main():
    stride, masks = {}, {}
    for name in MAPS:
        stride.update(stride_schedule(name))
    for name in MASKS:
        masks.update(mask_schedule(name))
    np.savez_compressed(os.path.join(HERE, "stride_schedules.npz"), **stride)
    np.savez_compressed(os.path.join(HERE, "mask_schedules.npz"), **masks)
    for fn in ("stride_schedules.npz", "mask_schedules.npz"):
        print(fn, os.path.getsize(os.path.join(HERE, fn)), "bytes")


if __name__ == "__main__":
    main()
