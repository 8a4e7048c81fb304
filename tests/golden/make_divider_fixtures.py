"""Writes ``tests/golden/divider_maps.npz``: the divider maps the REFERENCE's own code produces.

The one function of the path that nothing else pins is the mapping redundancy map -> divider map
(``RedundancyMap.generate_divider_map_from_redundancy`` followed by ``_refine_divider_map``,
core/redundancy_map.py:199-326, called in that order by ``init_redundancy_map`` :717-724): integer
logic on the percentiles of a measured map.  This script runs exactly those two functions, imported
from the reference tree, on the three redundancy maps the reference ships with the percentiles and
dividers of the three ``config.yaml`` files next to them, for ring sizes 2, 4, 8 and 16, and stores
inputs and outputs as plain arrays.  Nothing of the reference's text is kept, only those vectors.

It runs in the build container only (the reference tree is not available anywhere else); the
committed ``.npz`` is what the tests read.  The reference's files import each other under the
package name ``ditango``, so the tree is registered under that name; the class is instantiated
without its ``__init__`` (which asks a process group for the ring size) and given the ring size
directly.

    python tests/golden/make_divider_fixtures.py [/root/reference]
"""
import os
import sys
import types

import numpy as np
import torch
import yaml

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))
MODELS = {"cogvideox-5b": (50, 42), "hunyuanvideo": (50, 60), "stepvideo": (50, 48)}
RING_SIZES = (2, 4, 8, 16)


def main():
    pkg = types.ModuleType("ditango")
    pkg.__path__ = [REF]
    sys.modules["ditango"] = pkg
    from ditango.core import redundancy_map as ref  # the reference's module, unmodified

    out = {}
    for model, (T, L) in MODELS.items():
        base = os.path.join(REF, "configs", model)
        red = torch.load(os.path.join(base, f"redundancy_map_{T}_{L}.pt"), map_location="cpu", weights_only=True)
        with open(os.path.join(base, "config.yaml")) as f:
            cfg = yaml.safe_load(f)
        pct, div = list(cfg["stride-percentiles"]), list(cfg["stride-dividers"])
        assert tuple(red.shape) == (T, L)
        key = model.replace("-", "_")
        out[f"{key}.redundancy"] = red.to(torch.float32).numpy()
        out[f"{key}.percentiles"] = np.asarray(pct, dtype=np.int64)
        out[f"{key}.dividers"] = np.asarray(div, dtype=np.int64)
        for n in RING_SIZES:
            rm = object.__new__(ref.RedundancyMap)
            rm.num_timesteps, rm.num_layers, rm.base_weight = T, L, n
            rm.stride_divider, rm.map_percentage = [8, 4, 2, 1], [20, 50, 80]   # the class defaults (:32-33)
            rm.redundancy_map = red
            rm.divider_map = rm._init_map()
            thresholds = rm.generate_divider_map_from_redundancy(custom_percentages=pct, custom_dividers=div)
            out[f"{key}.N{n}.thresholds"] = np.asarray(thresholds, dtype=np.float64)
            out[f"{key}.N{n}.generated"] = rm.divider_map.numpy().astype(np.int64).copy()
            changes = rm._refine_divider_map()
            out[f"{key}.N{n}.refined"] = rm.divider_map.numpy().astype(np.int64).copy()
            out[f"{key}.N{n}.changes"] = np.asarray(changes, dtype=np.int64)
            print(f"{model} N={n}: thresholds {thresholds}, {changes} entries changed by the refinement,"
                  f" histogram {dict(zip(*np.unique(out[f'{key}.N{n}.refined'], return_counts=True)))}")
    path = os.path.join(HERE, "divider_maps.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
