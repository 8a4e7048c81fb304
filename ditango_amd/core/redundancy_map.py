"""Schedule source of the cached block attention: the redundancy map, the divider
map derived from it, and (an addition) an explicit per-chunk reuse mask.

API of the reference's ``core/redundancy_map.py``: class ``RedundancyMap`` and
the module functions ``init_redundancy_map``, ``get_redundancy_map``,
``save_redundancy_map``, ``save_divider_map``, ``is_preprocessing``,
``redundancy_preprocess``, ``generate_divider_map_with_custom_settings``,
``print_redundancy_map``.  The matplotlib visualisers of the reference
(:328-588) are cosmetic and are replaced by a text summary.

Stride mode (reference behaviour): ``divider_map[t, l]`` in {1,2,4,8} gives the
stride ``N // divider`` = how many KV chunks are recomputed at step ``t`` in
layer ``l`` (:49-87).

Mask mode (addition): ``set_chunk_mask(mask[T,L,C])`` installs a per-chunk
reuse mask; the compact compute/reuse lists of every ``(t, l)`` are built once
on the GPU by ``dt_build_schedule_table`` and stay in device memory, where the
attention kernel reads them.
"""
from __future__ import annotations

import os
from typing import List, Optional, Sequence

import numpy as np
import torch

from .. import _hip
from ..logger import init_logger
from ..utils import get_timestep
from .config import get_config
from .parallel_state import get_usp_group

logger = init_logger(__name__)


class RedundancyMap:
    def __init__(self, args):
        self.num_timesteps = args.num_inference_steps  # :27
        self.num_layers = args.num_layers  # :28
        self.base_weight = get_usp_group().world_size  # :29
        self.divider_map = self._init_map()
        self.stride_divider = [8, 4, 2, 1]  # :32
        self.map_percentage = [20, 50, 80]  # :33
        self.auto_setting = False
        self.calc_round = 0
        self.prev_out: List[Optional[torch.Tensor]] = [None] * self.num_layers
        self.redundancy_map: Optional[torch.Tensor] = None
        self._redundancy_dev: Optional[torch.Tensor] = None  # device-side accumulator while profiling
        # mask mode
        self.chunk_mask: Optional[np.ndarray] = None
        self.mask_diag: int = -1
        self.sched_compute_ids: Optional[torch.Tensor] = None  # int32 [T,L,C] device
        self.sched_reuse_ids: Optional[torch.Tensor] = None
        self.sched_counts: Optional[torch.Tensor] = None  # int32 [T,L,2] device
        self.sched_counts_host: Optional[np.ndarray] = None
        self.sched_windows: list = []  # (first chunk, end, diag in window, compute ids, counts, counts on host)

    # ---- divider map / strides ---------------------------------------------------------------
    def _init_map(self) -> torch.Tensor:
        return torch.ones(self.num_timesteps, self.num_layers, dtype=torch.long)

    def is_auto_setting(self) -> bool:
        return self.auto_setting

    def _stride_of(self, divider: int) -> int:
        if self.base_weight < divider:  # :63-64
            return 1
        assert self.base_weight % divider == 0, f"Invalid divider {divider} for base weight {self.base_weight}"
        return max(self.base_weight // divider, 1)

    def get_curr_isp_stride(self, timestep: int, layer_id: int) -> int:
        """:49-67"""
        if self.auto_setting:
            return self.base_weight
        return self._stride_of(int(self.divider_map[timestep, layer_id].item()))

    def get_next_isp_stride(self, timestep: int, layer_id: int) -> int:
        """:69-87 -- the last step announces a full refresh."""
        if self.auto_setting or timestep == self.num_timesteps - 1:
            return self.base_weight
        return self._stride_of(int(self.divider_map[timestep + 1, layer_id].item()))

    def set_pattern_for_row(self, row_idx: int, split_list: Sequence[int], pattern_list: Sequence[int]) -> None:
        """:90-119 -- piecewise-constant dividers over the layers of one step."""
        if row_idx >= self.num_timesteps:
            raise ValueError(f"Row index {row_idx} exceeds num_timesteps {self.num_timesteps}")
        if pattern_list is None or len(pattern_list) == 0:
            return
        split_list = list(split_list or [])
        assert len(split_list) + 1 == len(pattern_list), (
            f"Number of patterns does not match number of split chunks. Expected {len(split_list) + 1} patterns")
        bounds = [0] + split_list + [self.num_layers]
        for i, p in enumerate(pattern_list):
            assert p <= self.base_weight, f"isp size {p} should be less than osp size {self.base_weight}"
            self.divider_map[row_idx, bounds[i]:bounds[i + 1]] = p

    def set_pattern_for_rows(self, timestep_indices, split_list: Sequence[int] = (), pattern_list: Sequence[int] = ()) -> None:
        """:121-136"""
        if len(timestep_indices) == 0 or len(pattern_list) == 0:
            return
        for idx in list(timestep_indices):
            self.set_pattern_for_row(idx, split_list, pattern_list)

    def set_full_stride_for_rows(self, timestep_indices) -> None:
        """:138-149 (writes ``base_weight`` as the divider, i.e. stride 1, as the reference does)."""
        for idx in list(timestep_indices):
            self.set_pattern_for_row(idx, [], [self.base_weight])

    def get_map(self) -> torch.Tensor:
        return self.divider_map

    def reset_map(self) -> None:
        self.divider_map = self._init_map()

    # ---- profiling mode ------------------------------------------------------------------------
    def enable_auto_setting(self) -> None:
        """:160-172"""
        if get_timestep() != 0:
            logger.warning(f"Auto setting enabled at timestep {get_timestep()}, should be 0")
        self.auto_setting = True
        self.redundancy_map = torch.zeros(self.num_timesteps, self.num_layers, dtype=torch.float)
        self._redundancy_dev = None
        self.prev_out = [None] * self.num_layers
        logger.info("Auto setting enabled for RedundancyMap")

    def record_out_redundancy(self, timestep: int, layer_id: int, curr_out: torch.Tensor) -> None:
        """:174-197.  ``redundancy[t,l] += rel_l1(curr_out, prev_out)`` with the reduction
        (``dt_rel_l1_sums``) and the accumulation both on the device: no host sync per call."""
        if not self.auto_setting:
            return
        prev = self.prev_out[layer_id]
        if prev is None:
            self.prev_out[layer_id] = curr_out
            return
        if self._redundancy_dev is None:
            self._redundancy_dev = torch.zeros(self.num_timesteps, self.num_layers, dtype=torch.float64,
                                               device=curr_out.device)
        s = _hip.rel_l1_sums(curr_out.to(torch.float32).contiguous(), prev.to(torch.float32).contiguous())
        cnt = s[3]
        new_abs_mean = s[1] / cnt
        ori_abs_mean = s[2] / cnt
        val = (s[0] / cnt) / (ori_abs_mean + 1e-8)
        val = torch.where(ori_abs_mean < 1e-6, new_abs_mean, val)  # utils.py:236-238
        inf = torch.full_like(val, float("inf"))
        val = torch.where((cnt == 0) | torch.isnan(val), inf, val)  # utils.py:219-222, 262-265
        self._redundancy_dev[timestep, layer_id] += val
        self.prev_out[layer_id] = curr_out

    def _sync_redundancy(self) -> None:
        if self._redundancy_dev is not None:
            self.redundancy_map = self._redundancy_dev.to(torch.float32).cpu()

    def finished_one_round(self) -> None:
        """:590-596"""
        self.calc_round += 1
        self.prev_out = [None] * self.num_layers
        logger.info(f"Finished RedundancyMap auto-setting round {self.calc_round}")

    def finish_auto_setting(self) -> None:
        """:598-626.  The reference averages the map over all ranks with an all-reduce;
        one GPU plays one rank, so the map is this rank's own."""
        if not self.auto_setting:
            logger.info("Auto setting is not enabled, nothing to finish")
            return
        self._sync_redundancy()
        cfg = get_config()
        if cfg is None or cfg.rank == 0:
            try:
                save_redundancy_map(override=True)
            except Exception as e:  # saving is best effort, as in the reference (:798-800)
                logger.error(f"Failed to save redundancy map: {e}")
        self.auto_setting = False
        self.prev_out = [None] * self.num_layers

    # ---- redundancy -> dividers ---------------------------------------------------------------
    def generate_divider_map_from_redundancy(self, custom_percentages=None, custom_dividers=None):
        """:199-279"""
        if self.redundancy_map is None:
            logger.warning("Cannot generate divider map: no redundancy data available")
            return None
        percentages = custom_percentages if custom_percentages is not None else self.map_percentage
        dividers = custom_dividers if custom_dividers is not None else self.stride_divider
        red = self.redundancy_map.to(torch.float32).cpu().numpy().astype(np.float64)
        positive = red[red > 0]
        if positive.size == 0:
            logger.warning("No non-zero redundancy values found, keeping default divider map")
            return None
        percentiles = [float(np.percentile(positive, p)) for p in percentages]
        logger.info(f"Generating divider map with percentiles {percentiles} for percentages {percentages}, dividers {dividers}")
        # bin index 0..3 by the three thresholds, strict '<' as in the reference
        bins = (red >= percentiles[0]).astype(np.int64) + (red >= percentiles[1]) + (red >= percentiles[2])
        chosen = np.asarray(dividers, dtype=np.int64)[bins]
        valid_desc = sorted(dividers)
        fixed = np.empty_like(chosen)
        for d in np.unique(chosen):
            dd = int(d)
            if self.base_weight < dd:  # :262-263
                dd = self.base_weight
            elif self.base_weight % dd != 0:  # :264-271
                for cand in valid_desc:
                    if self.base_weight % cand == 0 and cand <= dd:
                        dd = cand
                        break
                else:
                    dd = 1
            fixed[chosen == d] = dd
        div = np.where(red > 0, fixed, 1)
        div[self.num_timesteps - 1, :] = 1  # :244-246
        self.divider_map = torch.from_numpy(div.astype(np.int64))
        logger.info("Divider map generation complete")
        return percentiles

    def _refine_divider_map(self):
        """:281-326 -- per layer, in step order, reading the already refined previous step."""
        if self.divider_map is None:
            logger.warning("Cannot refine divider map: map not initialized")
            return
        div = self.divider_map.cpu().numpy().copy()
        T = self.num_timesteps
        changes = 0
        for layer in range(self.num_layers):
            col = div[:, layer]
            for t in range(1, T):
                if t < 3 or t > T - 3:
                    new = 1
                elif col[t - 1] == 1 or col[t] <= col[t - 1]:
                    continue
                else:
                    new = 1
                if col[t] != new:
                    col[t] = new
                    changes += 1
        self.divider_map = torch.from_numpy(div)
        if changes > 0:
            logger.info(f"Refined divider map: {changes} values changed to ensure valid transitions")
        return changes

    # ---- text summaries in place of the reference's plots -----------------------------------
    def stride_table(self) -> np.ndarray:
        div = torch.clamp_max(self.divider_map, self.base_weight)
        return (self.base_weight // div).cpu().numpy()

    def visualize_divider_map(self, output_dir=None, file_prefix="stride"):
        """Writes ``<prefix>_info.txt`` (divider histogram + stride grid); no plots."""
        if output_dir is None:
            return None
        os.makedirs(output_dir, exist_ok=True)
        path = os.path.join(output_dir, f"{file_prefix}_info.txt")
        vals, counts = np.unique(self.divider_map.cpu().numpy(), return_counts=True)
        with open(path, "w") as f:
            f.write(f"timesteps {self.num_timesteps} layers {self.num_layers} base_weight {self.base_weight}\n")
            for v, c in zip(vals, counts):
                f.write(f"divider {int(v)}: {int(c)}\n")
            for row in self.stride_table():
                f.write(" ".join(f"{int(x):2d}" for x in row) + "\n")
        return [path]

    def visualize_redundancy_map(self, output_dir, file_prefix="redundancy"):
        return None

    # ---- mask mode -------------------------------------------------------------------------------
    def set_chunk_mask(self, mask, diag: Optional[int] = None, device=None) -> None:
        """Install a per-chunk reuse mask ``[T, L, C]`` (1 = reuse the cached state of
        chunk c, 0 = recompute).  ``diag`` is the local chunk, always recomputed and
        never cached; default = this rank's chunk; ``-1`` = none."""
        m = np.ascontiguousarray(np.asarray(mask, dtype=np.uint8))
        assert m.ndim == 3 and m.shape[0] == self.num_timesteps and m.shape[1] == self.num_layers, (
            f"mask must be [{self.num_timesteps},{self.num_layers},C], got {m.shape}")
        if diag is None:
            diag = get_usp_group().rank_in_group
        self.chunk_mask = m
        self.mask_diag = int(diag)
        dev = device if device is not None else torch.device("cuda", torch.cuda.current_device())
        dmask = torch.from_numpy(m).to(dev)
        comp, reu, cnt = _hip.build_schedule_table(dmask, self.mask_diag)
        self.sched_compute_ids, self.sched_reuse_ids, self.sched_counts = comp, reu, cnt
        self.sched_counts_host = cnt.cpu().numpy()  # one read-back at install time, none per call
        # One attention launch addresses at most DT_MAX_CHUNKS chunks: more chunks run as one launch per
        # window of chunk ids, each with its own compute list (ids relative to the window's first chunk).
        self.sched_windows = []
        C = m.shape[2]
        if C > _hip.DT_MAX_CHUNKS:
            for w0 in range(0, C, _hip.DT_MAX_CHUNKS):
                w1 = min(C, w0 + _hip.DT_MAX_CHUNKS)
                d_w = self.mask_diag - w0 if w0 <= self.mask_diag < w1 else -1
                c_w, _, n_w = _hip.build_schedule_table(dmask[:, :, w0:w1].contiguous(), d_w)
                self.sched_windows.append((w0, w1, d_w, c_w, n_w, n_w.cpu().numpy()))

    def clear_chunk_mask(self) -> None:
        self.chunk_mask = None
        self.sched_compute_ids = self.sched_reuse_ids = self.sched_counts = None
        self.sched_counts_host = None
        self.sched_windows = []


def make_bernoulli_mask(num_timesteps: int, num_layers: int, num_chunks: int, reuse_prob: float, seed: int,
                        diag: int = -1, cold_first_step: bool = True) -> np.ndarray:
    """Seeded per-chunk reuse mask ``[T, L, C]`` uint8: entry = 1 with probability
    ``reuse_prob`` (``numpy.random.default_rng(seed).random() < reuse_prob``); the local
    chunk ``diag`` is never reused and step 0 reuses nothing (the cache is cold)."""
    rng = np.random.default_rng(seed)
    m = (rng.random((num_timesteps, num_layers, num_chunks)) < reuse_prob).astype(np.uint8)
    if 0 <= diag < num_chunks:
        m[:, :, diag] = 0
    if cold_first_step:
        m[0] = 0
    return m


def print_redundancy_map(logger_=None):
    """:628-658"""
    rm = get_redundancy_map()
    if rm is None:
        print("Stride map not initialized", flush=True)
        return
    text = "\n".join(" ".join(f"{int(x):2d}" for x in row) for row in rm.stride_table())
    msg = f"===== DiTango Stride Map =====\n{text}\n================================="
    cfg = get_config()
    if cfg is None or cfg.rank == 0:
        (logger_.info if logger_ else print)(msg)


_redundancy_map: Optional[RedundancyMap] = None


def _default_map_path(args) -> str:
    return os.path.join(f"{args.ditango_base}/configs/{args.model_name}/",
                        f"redundancy_map_{args.num_inference_steps}_{args.num_layers}.pt")


def init_redundancy_map(args, redun_map_path=None, custom_percentages=None, custom_dividers=None, quiet=False):
    """:662-748"""
    global _redundancy_map
    assert _redundancy_map is None, "Stride map is already initialized"
    rm = RedundancyMap(args)
    _redundancy_map = rm
    if custom_percentages is None and hasattr(args, "stride_percentiles"):
        custom_percentages = args.stride_percentiles
    if custom_dividers is None and hasattr(args, "stride_dividers"):
        custom_dividers = args.stride_dividers
    if getattr(args, "use_pab", False):
        if not quiet:
            print_redundancy_map()
        return rm
    if redun_map_path is None:
        default_path = _default_map_path(args)
        if os.path.exists(default_path):
            redun_map_path = default_path
        else:
            logger.warning(f"No pre-computed redundancy map found at default location: {default_path}, Using full stride map instead")
    if redun_map_path is not None and os.path.exists(redun_map_path):
        try:
            loaded = torch.load(redun_map_path, map_location="cpu", weights_only=True)
            if loaded.shape[0] == args.num_inference_steps and loaded.shape[1] == args.num_layers:
                rm.redundancy_map = loaded
                rm.generate_divider_map_from_redundancy(custom_percentages=custom_percentages,
                                                        custom_dividers=custom_dividers)
                rm._refine_divider_map()
                logger.info(f"Successfully loaded redundancy map with shape {tuple(loaded.shape)}")
            else:
                logger.warning(f"Loaded map dimensions {tuple(loaded.shape)} don't match required dimensions "
                               f"({args.num_inference_steps}, {args.num_layers}). Using default map instead.")
        except Exception as e:
            logger.warning(f"Failed to load redundancy map: {e}. Using default map instead.")
    if not quiet:
        print_redundancy_map()
    return rm


def destroy_redundancy_map() -> None:
    global _redundancy_map
    _redundancy_map = None


def save_redundancy_map(path=None, override=False):
    """:750-800"""
    args = get_config()
    rm = get_redundancy_map()
    if rm is None or rm.redundancy_map is None:
        logger.warning("Cannot save redundancy map: stride map not initialized or no redundancy data available")
        return None
    if args is not None and args.rank != 0:
        return None
    if path is None:
        path = _default_map_path(args)
    if os.path.exists(path) and not override:
        logger.warning(f"File {path} already exists. Use override=True to replace it.")
        return None
    os.makedirs(os.path.dirname(path) or ".", exist_ok=True)
    torch.save(rm.redundancy_map, path)
    logger.info(f"Redundancy map saved to {path}")
    return path


def save_divider_map(path=None, override=False):
    """:802-845"""
    args = get_config()
    rm = get_redundancy_map()
    if rm is None:
        logger.warning("Cannot save divider map: stride map not initialized")
        return None
    if args is not None and args.rank != 0:
        return None
    if path is None:
        path = os.path.join(f"{args.ditango_base}/configs/{args.model_name}/",
                            f"divider_map_{rm.num_timesteps}_{rm.num_layers}.pt")
    if os.path.exists(path) and not override:
        logger.warning(f"File {path} already exists. Use override=True to replace it.")
        return None
    os.makedirs(os.path.dirname(path) or ".", exist_ok=True)
    torch.save(rm.divider_map, path)
    logger.info(f"Divider map saved to {path}")
    return path


def get_redundancy_map() -> Optional[RedundancyMap]:
    return _redundancy_map


def is_preprocessing() -> bool:
    return _redundancy_map is not None and _redundancy_map.auto_setting


def redundancy_preprocess(func, func_args, prompt_list=None):
    """:863-900 -- run the generation callable once per prompt with profiling on.
    (The reference reads ``prompt_list`` before assigning it and raises; here it is
    an optional argument with the same three default prompts' role.)"""
    if prompt_list is None:
        prompt_list = [
            "A playful black Labrador in a pumpkin costume frolics in a sunlit autumn garden.",
            "A boat glides along the Seine with the Eiffel Tower in the background, oil painting.",
            "A cat walks on the grass, realistic style.",
        ]
    rm = get_redundancy_map()
    rm.enable_auto_setting()
    for prompt in prompt_list:
        func(prompt=prompt, **func_args)
        rm.finished_one_round()
    rm.finish_auto_setting()


def generate_divider_map_with_custom_settings(custom_percentages=None, custom_dividers=None, output_dir=None):
    """:904-956"""
    rm = get_redundancy_map()
    if rm is None or rm.redundancy_map is None:
        logger.warning("Cannot generate custom divider map: stride map not initialized or no redundancy data")
        return None
    config = get_config()
    if config is not None and config.rank != 0:
        return None
    if custom_percentages is None:
        custom_percentages = config.stride_percentiles
    if custom_dividers is None:
        custom_dividers = config.stride_dividers
    rm.generate_divider_map_from_redundancy(custom_percentages=custom_percentages, custom_dividers=custom_dividers)
    rm._refine_divider_map()
    pct = "_".join(str(p) for p in custom_percentages)
    dvs = "_".join(str(d) for d in custom_dividers)
    return rm.visualize_divider_map(output_dir=output_dir, file_prefix=f"stride_custom_p{pct}_d{dvs}")
