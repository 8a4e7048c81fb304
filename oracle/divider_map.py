"""Redundancy map -> divider map -> strides (CPU oracle; test infrastructure only).

Restates ``RedundancyMap.generate_divider_map_from_redundancy``
(core/redundancy_map.py:199-279), ``_refine_divider_map`` (:281-326) and the
stride lookups (:49-87) on plain numpy arrays.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import numpy as np


def generate_divider_map(redundancy: np.ndarray, base_weight: int,
                         percentages: Sequence[float] = (20, 50, 80),
                         dividers: Sequence[int] = (8, 4, 2, 1)) -> Tuple[np.ndarray, Optional[List[float]]]:
    """core/redundancy_map.py:199-279.

    ``redundancy`` fp32 ``[T,L]``.  Returns (int64 divider map ``[T,L]``,
    percentile values).  Defaults for ``percentages``/``dividers`` are the class
    defaults (:32-33).  If no entry is positive the map stays all ones (:226-228).
    """
    T, L = redundancy.shape
    div = np.ones((T, L), dtype=np.int64)  # _init_map, :41-43
    # :219-224 python floats of the fp32 entries (``.item()``)
    vals = [float(redundancy[t, l]) for t in range(T) for l in range(L) if float(redundancy[t, l]) > 0]
    if len(vals) == 0:
        return div, None
    nz = np.array(vals)
    pct = [float(np.percentile(nz, p)) for p in percentages]  # :232 (linear interpolation)
    for t in range(T):
        for l in range(L):
            if t == T - 1:  # :244-246
                div[t, l] = 1
                continue
            red = float(redundancy[t, l])
            if red > 0:  # :250
                if red < pct[0]:
                    d = dividers[0]
                elif red < pct[1]:
                    d = dividers[1]
                elif red < pct[2]:
                    d = dividers[2]
                else:
                    d = dividers[3]
                if base_weight < d:  # :262-263
                    d = base_weight
                elif base_weight % d != 0:  # :264-271
                    for cand in sorted(dividers):
                        if base_weight % cand == 0 and cand <= d:
                            d = cand
                            break
                    else:
                        d = 1
                div[t, l] = int(d)
    return div, pct


def refine_divider_map(div: np.ndarray) -> Tuple[np.ndarray, int]:
    """core/redundancy_map.py:281-326.  Sequential per layer: step ``t`` reads
    the ALREADY refined value of step ``t-1`` (:300-301 read the live map)."""
    out = div.copy()
    T, L = out.shape
    for layer in range(L):
        for t in range(1, T):
            cur = int(out[t, layer])
            prev = int(out[t - 1, layer])
            if t < 3 or t > T - 3:  # :302-304
                out[t, layer] = 1
                continue
            if prev == 1:  # :308-310
                continue
            if cur <= prev:  # :313-315
                continue
            out[t, layer] = 1  # :319
    changes = int((out != div).sum())
    return out, changes


def curr_stride(div: np.ndarray, base_weight: int, t: int, layer: int, auto_setting: bool = False) -> int:
    """core/redundancy_map.py:49-67."""
    if auto_setting:
        return base_weight
    d = int(div[t, layer])
    if base_weight < d:
        return 1
    assert base_weight % d == 0, f"Invalid divider {d} for base weight {base_weight}"
    return max(base_weight // d, 1)


def next_stride(div: np.ndarray, base_weight: int, t: int, layer: int, auto_setting: bool = False) -> int:
    """core/redundancy_map.py:69-87."""
    T = div.shape[0]
    if auto_setting or t == T - 1:
        return base_weight
    d = int(div[t + 1, layer])
    if base_weight < d:
        return 1
    assert base_weight % d == 0, f"Invalid divider {d} for base weight {base_weight}"
    return base_weight // d
