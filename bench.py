#!/usr/bin/env python3
"""Benchmark of the cached block attention hot path on ONE MI355X.

A "step" is one ``proAttention.attn`` call (one transformer layer's attention at one
diffusion step) at the HunyuanVideo per-rank shape: local query shard of 14882 tokens,
KV = 8 chunks of 14882 tokens, H=24, D=128, bf16, under the seeded Bernoulli(0.6) reuse mask
over 50 steps x 60 layers.  Inputs are resident in HBM before the timed region.

The timed calls are a stratified sample of the schedule's (step, layer) rows: the rows are grouped by
the number of chunks they recompute and the next row always comes from the group that is furthest
behind its share, so any number of steps sees the schedule's mix of cheap and expensive rows and
``value`` does not depend on ``--steps``.

Prints ONE JSON line: ms per layer call plus
  * ``roofline``        the fresh-chunk attention kernel against the bf16 dense MFMA peak,
  * ``roofline_merge``  the fused LSE-merge kernel against the HBM peak,
  * ``cache_gbs``       cache store / load copies against the HBM peak,
  * ``launch_floor``    empty kernels of the merge's and the copy's grids (what a short launch pays before it moves a byte),
  * ``varlen``          the variable-length entry with its cu_seqlens on the GPU, as the model passes them,
  * ``other_configs``   compact records of the other single-GPU configurations (CogVideoX share,
                        Step-Video share, the 32-chunk reuse sweep) and ``stride_schedule``: one full pass of the
                        reference's own stride schedule from the HunyuanVideo redundancy map it ships,
  * ``cpu_baseline``    the torch-math oracle timed on this box's host cores on a bounded sample.
The HBM-bound kernels are timed over a rotation of distinct buffers of more than 1 GB in total,
so the figures are those of HBM and not of the 256 MB memory-side cache.
"""
import argparse
import json
import math
import os
import subprocess
import sys
import threading
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import bench_probes  # noqa: E402  (the measurement aids live beside this file, outside the package)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E
NOMINAL_CLOCK_MHZ = 2400.0  # the shader clock the bf16 peak is quoted at

WORKLOADS = {
    # name: (label, B, H, D, Sq, chunk lengths, T, L, reuse probability, diag, qk norm)
    "hunyuanvideo": ("HunyuanVideo per-rank share (configs[2])", 1, 24, 128, 14882, [14882] * 8, 50, 60, 0.6, 0, "rms"),
    "cogvideox": ("CogVideoX-5B per-rank share (configs[1])", 1, 48, 64, 2222, [2222] * 8, 50, 42, 0.5, 0, "layer"),
    "stepvideo": ("Step-Video-T2V per-rank share (configs[3])", 1, 48, 128, 6851, [6851] * 8, 50, 48, 0.75, 0, None),
    "sweep": ("reuse sweep at HunyuanVideo scale (configs[4])", 1, 24, 128, 119056, [3721] * 16 + [3720] * 16, 1, 60, 0.5, -1, "rms"),
}


def make_inputs(B, H, D, Sq, lens, norm, device, seed=0):
    """Seeded synthetic q / K chunks / V chunks, drawn on the device (Q and K normalised over D as the model does)."""
    g = torch.Generator(device=device).manual_seed(seed)

    def draw(n, normalise):
        x = torch.randn(B, n, H, D, generator=g, device=device)
        if normalise == "rms":
            x = x / x.pow(2).mean(-1, keepdim=True).sqrt()
        elif normalise == "layer":
            x = torch.nn.functional.layer_norm(x, (D,))
        return x.bfloat16()

    q = draw(Sq, norm)
    ks = [draw(n, norm) for n in lens]
    vs = [draw(n, None) for n in lens]
    return q, ks, vs


PROFILING = False   # --kernels-only: a handful of launches per kernel, no minimum timed duration


def time_kernel(fn, reps, warm=3, min_ms=40.0):
    """Average duration in ms of ``fn`` over ``reps`` launches (HIP events on the launch stream)."""
    if PROFILING:
        warm, reps, min_ms = 1, 2, 0.0
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    total = e0.elapsed_time(e1)
    if total < min_ms:  # short kernels: time at least min_ms of them, so that clock ramps average out
        more = int(reps * min_ms / max(total, 1e-3)) + 1
        e0.record()
        for _ in range(more):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / more
    return total / reps


class Rotation:
    """Calls ``fn(i)`` with i cycling through ``n`` argument sets (distinct memory per call)."""

    def __init__(self, fn, n):
        self.fn, self.n, self.k = fn, max(1, n), 0

    def __call__(self):
        self.fn(self.k % self.n)
        self.k += 1


def _hwmon_watts(name):
    """The first readable ``power1_<name>`` of a GPU's hwmon node, in W (the files hold microwatts), or None."""
    import glob
    for path in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_" + name)):
        try:
            with open(path) as f:
                return int(f.read().strip()) / 1e6
        except (OSError, ValueError):
            continue
    return None


def sample_clock_and_power(fn, seconds=2.0):
    """(shader clock in MHz from ``rocm-smi``, package power in W from the GPU's hwmon node) while ``fn`` keeps the
    GPU busy; None for what cannot be read."""
    clocks, watts, stop = [], [], [False]

    def sampler():
        while not stop[0]:
            try:
                w = _hwmon_watts("input")
                if w is None:
                    w = _hwmon_watts("average")
                if w is not None:
                    watts.append((time.perf_counter(), w))
                r = subprocess.run(["rocm-smi", "--showclocks", "--json"], capture_output=True, text=True, timeout=10)
                card = list(json.loads(r.stdout[r.stdout.index("{"):]).values())[0]
                clocks.append((time.perf_counter(), float(card["sclk clock speed:"].strip("()Mhz"))))
            except Exception:
                pass
            time.sleep(0.1)

    th = threading.Thread(target=sampler, daemon=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    th.start()
    while time.perf_counter() - t0 < seconds:
        for _ in range(4):
            fn()
        torch.cuda.synchronize()
    stop[0] = True
    th.join(timeout=15)

    def mean(samples):
        vals = [v for ts, v in samples if ts - t0 > 0.5]   # after the ramp
        return round(sum(vals) / len(vals), 0) if vals else None
    return mean(clocks), mean(watts)


def sample_clock_mhz(fn, seconds=2.0):
    return sample_clock_and_power(fn, seconds)[0]


def power_cap_w():
    """The package power limit of the GPU's hwmon node in W, or None."""
    return _hwmon_watts("cap")


def stratified_order(counts):
    """A fixed visiting order of the schedule rows in which every prefix has (as nearly as whole rows allow)
    the whole schedule's distribution of ``counts``: the rows are grouped by count, and the next row always
    comes from the group that is furthest behind its share of the schedule (ties: the group nearest the
    mean); inside a group the rows are taken with a stride of about 1/golden-ratio of its size."""
    groups = {}
    for i, c in enumerate(counts):
        groups.setdefault(c, []).append(i)
    m = len(counts)
    mean = sum(counts) / max(m, 1)
    for c, rows in groups.items():
        n = len(rows)
        stride = max(1, int(n * 0.6180339887))
        while math.gcd(stride, n) != 1:
            stride += 1
        groups[c] = [rows[(j * stride) % n] for j in range(n)]
    taken = {c: 0 for c in groups}
    order = []
    for j in range(m):
        best = max((c for c in groups if taken[c] < len(groups[c])),
                   key=lambda c: (len(groups[c]) / m * (j + 1) - taken[c], -abs(c - mean)))
        order.append(groups[best][taken[best]])
        taken[best] += 1
    return order


def cpu_baseline(B, H, D, Sq, lens, mean_computed, n_chunks, norm, budget_s=20.0):
    """The oracle's torch math on the host cores, on a bounded sample scaled to one layer call."""
    from oracle import attention_math as om
    cores = len(os.sched_getaffinity(0))
    torch.set_num_threads(cores)
    Sk = lens[0]
    g = torch.Generator().manual_seed(1)
    heads = 1
    q = torch.randn(B, Sq, heads, D, generator=g).bfloat16()
    k = torch.randn(B, Sk, heads, D, generator=g).bfloat16()
    v = torch.randn(B, Sk, heads, D, generator=g).bfloat16()
    t0 = time.perf_counter()
    n_done = 0
    while True:
        om.chunk_attention(q, k, v)
        n_done += 1
        el = time.perf_counter() - t0
        if el > budget_s * 0.7 or n_done >= 32:
            break
    per_head_chunk = el / n_done
    # merge of n_chunks states on 1/8 of the rows, literal reference fold
    rows_s = max(1, Sq // 8)
    outs = [torch.randn(B, rows_s, H, D, generator=g).bfloat16() for _ in range(n_chunks)]
    lses = [torch.randn(B, H, rows_s, generator=g) for _ in range(n_chunks)]
    t1 = time.perf_counter()
    o = l = None
    for bo, bl in zip(outs, lses):
        o, l = om.update_out_and_lse(o, l, bo, bl)
    merge_s = (time.perf_counter() - t1) * (Sq / rows_s)
    layer_ms = 1e3 * (per_head_chunk * H * mean_computed + merge_s)
    flops = 4.0 * B * H * Sq * Sk * D * mean_computed
    return {
        "value": round(layer_ms, 1), "unit": "ms", "cores": cores, "kind": "port",
        "attn_tflops": round(flops / (per_head_chunk * H * mean_computed) / 1e12, 3),
        "sample": (f"{n_done}x one head of one KV chunk (Sq={Sq}, Sk={Sk}, D={D}) in {el:.1f}s, scaled x{H} heads x "
                   f"{mean_computed:.2f} computed chunks/call; literal update_out_and_lse fold of {n_chunks} states on "
                   f"1/8 of the rows scaled x8"),
    }


def stride_schedule_record(n_layers):
    """One full pass of the reference's own schedule (core/attention.py:100-216, core/cache.py:28-72): 50 steps x
    ``n_layers`` layers of ``proAttention.attn`` at the HunyuanVideo per-rank shape as ring rank 0 of 8, with the
    divider map generated from the redundancy map the reference ships for HunyuanVideo (percentiles [0,40,90],
    dividers [8,4,2,1], configs/hunyuanvideo/config.yaml).  Every call is timed, the full-stride steps included.
    The in-place cache coarsening (``proCache._merge_blocks``) is bracketed by events of its own."""
    from ditango_amd.core import config, parallel_state, redundancy_map as rmod
    from ditango_amd.core.attention import proAttention
    from ditango_amd.utils import update_timestep
    label, B, H, D, Sq, lens, T, L, _, _, norm = WORKLOADS["hunyuanvideo"]
    N, rank = len(lens), 0
    L_run = min(L, n_layers)
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    parallel_state.init_local_groups(N, rank)
    cfg = config.init_config(None, num_inference_steps=T, num_layers=L, stride_percentiles=[0, 40, 90],
                             stride_dividers=[8, 4, 2, 1])
    rmod.destroy_redundancy_map()
    rmod.init_redundancy_map(cfg, redun_map_path=os.path.join(ROOT, "tests", "golden", "redundancy_map_50_60.pt"), quiet=True)
    q, ks, vs = make_inputs(B, H, D, Sq, lens, norm, dev)
    group = parallel_state.get_usp_group()
    group.set_kv_chunks(ks, vs)
    layers = [proAttention(l, group) for l in range(L_run)]
    coarsen_events = []

    def bracketed(merge_blocks):
        def run(new_block_num):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            merge_blocks(new_block_num)
            e1.record()
            coarsen_events.append((e0, e1))
        return run

    for layer in layers:
        layer.cache._merge_blocks = bracketed(layer.cache._merge_blocks)
    computed = reused = double_counted = 0
    strides = {}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for t in range(T):
        update_timestep(t)
        for l in range(L_run):
            layers[l].attn(q, ks[rank], vs[rank])
            plan = layers[l].last_plan
            computed += len(plan.computed)
            reused += len(plan.reuse_merged)
            double_counted += len(plan.computed) - len({c for c, _ in plan.computed})
            strides[plan.curr_stride] = strides.get(plan.curr_stride, 0) + 1
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    coarsen_ms = sum(e0.elapsed_time(e1) for e0, e1 in coarsen_events)
    calls = T * L_run
    flops = 4.0 * B * H * Sq * lens[0] * D * computed
    rmod.destroy_redundancy_map()
    parallel_state.destroy_local_groups()
    update_timestep(0)
    for layer in layers:
        layer.cache.release()
    del layers, q, ks, vs
    torch.cuda.empty_cache()
    return {
        "config": {"workload": label + ", stride schedule of the shipped redundancy map (refined dividers), ring rank 0 of 8",
                   "B": B, "H": H, "D": D, "Sq": Sq, "kv_chunks": N, "Sk": lens[0], "layers_instantiated": L_run,
                   "steps_per_layer": T, "calls_by_stride": {str(k): v for k, v in sorted(strides.items())}},
        "ms_per_layer": round(1e3 * elapsed / calls, 4), "calls": calls,
        "mean_chunks_computed_per_call": round(computed / calls, 3),
        "mean_cached_blocks_merged_per_call": round(reused / calls, 3),
        "calls_with_the_local_chunk_merged_twice": double_counted,
        "layer_attn_tflops": round(flops / elapsed / 1e12, 1),
        "coarsening": {"what": "in-place merges of proCache._merge_blocks, device time between events",
                       "launch_groups": len(coarsen_events), "ms_total": round(coarsen_ms, 3),
                       "share_of_run": round(coarsen_ms / (1e3 * elapsed), 5)},
    }


def bench_stride_schedule(args):
    """``--schedule stride``: the stride-schedule pass as a report of its own (default 12 layers)."""
    rec = stride_schedule_record(args.layers or 12)
    print(json.dumps({
        "metric": "ms/layer", "value": rec["ms_per_layer"], "unit": "ms", "n_gpus": 1, "steps": rec["calls"], "warmup": 0,
        "ms_per_step": rec["ms_per_layer"], "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic", **{k: v for k, v in rec.items() if k not in ("ms_per_layer", "calls")},
    }), flush=True)


def bench_item_model(args):
    """``--item-model``: what a work item of the attention kernel costs on top of its key tiles.  Launches whose
    items exactly fill the chip's workgroup slots (256 at D = 128, 512 at D = 64: 8 query tiles x 32 / 64 heads), with
    1, 2 and 4 rounds of such items (the same chunk as several jobs) and 8 ... 233 key tiles per item; prints the
    launches and the least-squares fit  round time = item cost + tile time x tiles  over the rounds after the first."""
    from ditango_amd import _hip
    dev = torch.device("cuda", 0)
    out = {"metric": "attention work-item cost model", "unit": "us", "n_gpus": 1, "dtype": "bf16", "data": "synthetic", "fits": {}}
    for D, heads, tiles_list in ((64, 64, (8, 16, 35, 70)), (128, 32, (8, 16, 59, 117, 233))):
        B, Sq = 1, 2048
        q = torch.randn(B, Sq, heads, D, device=dev).bfloat16()
        rows = []
        for tiles in tiles_list:
            Sk = tiles * 64
            k = torch.randn(B, Sk, heads, D, device=dev).bfloat16()
            v = torch.randn(B, Sk, heads, D, device=dev).bfloat16()
            table = _hip.ChunkTable([k], [v])
            o = torch.empty_like(q)
            l = torch.empty(B, heads, Sq, device=dev)
            per_rounds = {}
            for rounds in (1, 2, 4):
                ms = min(time_kernel(lambda: _hip.attn_jobs_fwd(q, table, [[0]] * rounds, [o] * rounds, [l] * rounds),
                                     args.kernel_reps) for _ in range(3))
                per_rounds[rounds] = ms * 1e3
            later = (per_rounds[4] - per_rounds[1]) / 3.0         # one round behind the first
            rows.append({"tiles": tiles, "us_1_round": round(per_rounds[1], 1), "us_2_rounds": round(per_rounds[2], 1),
                         "us_4_rounds": round(per_rounds[4], 1), "us_per_later_round": round(later, 2),
                         "first_round_extra_us": round(per_rounds[1] - later, 2)})
        x = np.array([r["tiles"] for r in rows], dtype=np.float64)
        y = np.array([r["us_per_later_round"] for r in rows], dtype=np.float64)
        slope, icpt = np.polyfit(x, y, 1)
        items = heads * (Sq // 256)
        flop_tile_round = 4.0 * items * 256 * 64 * D
        out["fits"][f"D{D}"] = {"items_per_round": items, "launches": rows, "tile_us": round(float(slope), 3),
                                "item_cost_us": round(float(icpt), 2), "item_cost_tiles": round(float(icpt / slope), 2),
                                "steady_state_tflops": round(flop_tile_round / (slope * 1e-6) / 1e12, 1),
                                "max_fit_error": round(float(np.max(np.abs(slope * x + icpt - y) / y)), 4)}
    print(json.dumps(out), flush=True)


def load_traffic(workload):
    """HBM bytes per launch from rocprofv3 FETCH_SIZE / WRITE_SIZE runs, committed under profiles/
    (``{"attn_fwd": {"<chunks per launch>": bytes, ...}, "merge_states": {"<states>": bytes}}``)."""
    path = os.path.join(ROOT, "profiles", f"hbm_traffic_{workload}.json")
    if not os.path.exists(path):
        return {}
    with open(path) as f:
        return json.load(f).get("bytes_per_launch", {})


def run_workload(name, args, steps, warmup, main, reuse=None, kernels_only=False):
    """Layer calls plus per-kernel launches of one workload; returns the record (main: the full one)."""
    from ditango_amd import _hip
    from ditango_amd.core import config, parallel_state, redundancy_map as rmod
    from ditango_amd.core.attention import proAttention
    from ditango_amd.utils import update_timestep

    label, B, H, D, Sq, lens, T, L, p, diag, norm = WORKLOADS[name]
    if reuse is not None:
        p = reuse
    C = len(lens)
    L_run = min(L, args.layers) if args.layers else L
    if name == "sweep":
        L_run = min(L_run, 2)   # 32 cached states of 743 MB per layer
        T = 2                   # step 0 fills the cache, step 1 is measured
    dev = torch.device("cuda", 0)
    rank = max(diag, 0)
    parallel_state.init_local_groups(C, rank)
    cfg = config.init_config(None, num_inference_steps=T, num_layers=L)
    rmod.destroy_redundancy_map()
    rmod._redundancy_map = rmod.RedundancyMap(cfg)
    rm = rmod.get_redundancy_map()
    mask = rmod.make_bernoulli_mask(T, L, C, p, seed=0, diag=diag)
    rm.set_chunk_mask(mask, diag=diag)

    q, ks, vs = make_inputs(B, H, D, Sq, lens, norm, dev)
    group = parallel_state.get_usp_group()
    group.set_kv_chunks(ks, vs)
    layers = [proAttention(l, group) for l in range(L_run)]

    # fill the caches: step 0 recomputes everything (not timed, not a warm-up step)
    update_timestep(0)
    for l in range(L_run):
        layers[l].attn(q, ks[rank], vs[rank])
    torch.cuda.synchronize()

    rows_tl = [(t, l) for t in range(1, T) for l in range(L_run)]
    counts = [int(rm.sched_counts_host[t, l, 0]) for t, l in rows_tl]
    order = stratified_order(counts)
    population_mean = float(np.mean(counts))
    seq = [rows_tl[order[i % len(order)]] for i in range(warmup + steps)]

    def run(t, l):
        update_timestep(t)
        return layers[l].attn(q, ks[rank], vs[rank])

    timed = seq[warmup:]
    if kernels_only:
        warmup, steps, timed = 0, 1, seq[:1]
    for t, l in seq[:warmup]:
        run(t, l)
    torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(len(timed) + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i, (t, l) in enumerate(timed):
        run(t, l)
        marks[i + 1].record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = 1e3 * elapsed / steps
    n_comp = [int(rm.sched_counts_host[t, l, 0]) for t, l in timed]
    mean_computed = float(np.mean(n_comp))
    # per-call device time by the number of chunks a call recomputes, and the mean over the WHOLE schedule it implies
    per_count = {}
    for i, k in enumerate(n_comp):
        per_count.setdefault(k, []).append(marks[i].elapsed_time(marks[i + 1]))
    hist = {k: counts.count(k) / len(counts) for k in set(counts)}
    covered = sum(w for k, w in hist.items() if k in per_count)
    schedule_mean_ms = sum(w * float(np.mean(per_count[k])) for k, w in hist.items() if k in per_count) / max(covered, 1e-9)
    Sk_mean = float(np.mean(lens))
    flops_per_chunk = 4.0 * B * H * Sq * Sk_mean * D
    rows = B * Sq * H

    # ---- per-kernel rooflines, measured live with HIP events on the launch stream ----------
    reps = args.kernel_reps if main else max(5, args.kernel_reps // 2)
    state_bytes = rows * (2 * D + 4)
    # the dominant kernel in its typical launch: as many single-chunk states as a layer call
    # computes on average over the schedule (rounded), written into cache-form states, one launch
    n_typ = max(1, min(C, int(round(population_mean))))
    table = _hip.ChunkTable(ks, vs)
    k1_ws = _hip.attn_workspace(dev)   # the launch as proAttention makes it: with the tail-balancing workspace
    st_outs = [torch.empty(B, Sq, H, D, dtype=torch.bfloat16, device=dev) for _ in range(n_typ)]
    st_lses = [torch.empty(B, H, Sq, dtype=torch.float32, device=dev) for _ in range(n_typ)]

    def k1_launch(n, qq=q, pre=False):
        _hip.attn_jobs_fwd(qq, table, [[c] for c in range(n)], st_outs[:n], st_lses[:n], workspace=k1_ws, q_prescaled=pre)

    def k1_flops(n):
        return sum(4.0 * B * H * Sq * lens[c] * D for c in range(n))

    if kernels_only:   # one launch of every size up to the chunk count, for the profiler (first dispatches of the kernel)
        st_outs += [torch.empty_like(st_outs[0]) for _ in range(C - n_typ)]
        st_lses += [torch.empty_like(st_lses[0]) for _ in range(C - n_typ)]
        for n in range(1, C + 1):
            k1_launch(n)
        torch.cuda.synchronize()
    k1_ms = time_kernel(lambda: k1_launch(n_typ), reps)
    k1_tflops = k1_flops(n_typ) / (k1_ms * 1e-3) / 1e12
    k1s_ms = time_kernel(lambda: k1_launch(1), reps)
    k1s_tflops = k1_flops(1) / (k1s_ms * 1e-3) / 1e12
    # the same typical launch in the opt-in mode of a caller that folds softmax_scale * log2(e) into q
    # (reported beside the drop-in figure, never in place of it)
    q_folded = (q.float() * (D ** -0.5 * math.log2(math.e))).to(torch.bfloat16)
    k1p_ms = time_kernel(lambda: k1_launch(n_typ, q_folded, True), reps)
    k1p_tflops = k1_flops(n_typ) / (k1p_ms * 1e-3) / 1e12
    # the same typical launch on IEEE-half copies of the tensors (a model run in fp16: fp16 MFMA, fp16 states)
    qh, ksh, vsh = q.half(), [k.half() for k in ks[:n_typ]], [v.half() for v in vs[:n_typ]]
    table_h = _hip.ChunkTable(ksh, vsh)
    sth = [torch.empty(B, Sq, H, D, dtype=torch.float16, device=dev) for _ in range(n_typ)]
    k1h_ms = time_kernel(lambda: _hip.attn_jobs_fwd(qh, table_h, [[c] for c in range(n_typ)], sth, st_lses[:n_typ], workspace=k1_ws), reps)
    k1h_tflops = k1_flops(n_typ) / (k1h_ms * 1e-3) / 1e12
    del qh, ksh, vsh, table_h, sth
    clock = watts = None
    mfma_probe = None
    if main and not kernels_only:
        clock, watts = sample_clock_and_power(lambda: k1_launch(n_typ))
        # the yardstick: back-to-back MFMAs on registers in the same launch shape, sized to last about as long
        # as the typical launch -- what the power limit leaves of the nominal peak when only the matrix pipes work
        probe_sink = torch.zeros(1, dtype=torch.float32, device=dev)
        probe_wgs, probe_iters = 256 * 8, 8192
        probe_flops = [0.0]

        def probe_launch():
            probe_flops[0] = bench_probes.mfma_probe(probe_wgs, probe_iters, probe_sink)

        kp_ms = time_kernel(probe_launch, reps)
        probe_clock, probe_watts = sample_clock_and_power(probe_launch, seconds=1.5)
        mfma_probe = {"tflops": round(probe_flops[0] / (kp_ms * 1e-3) / 1e12, 1), "launch_ms": round(kp_ms, 4),
                      "clock_mhz_under_load": probe_clock, "power_w_under_load": probe_watts}
    del q_folded
    # the co-issue yardstick: one wavefront of each SIMD issues MFMAs, the other the softmax's vector instructions
    # per MFMA at this head dimension; the MFMA rate with the softmax against the rate without is the ceiling of the
    # attention kernel's MFMA utilisation before any LDS traffic, barrier or tile load
    coissue = None
    if not kernels_only:
        co_sink = torch.zeros(1, dtype=torch.float32, device=dev)
        co_wgs, co_iters = 256 * 8, 4096
        co_flops = [0.0]

        def co_launch(with_softmax):
            co_flops[0] = bench_probes.coissue_probe(co_wgs, co_iters, D, with_softmax, co_sink)

        co0_ms = time_kernel(lambda: co_launch(False), reps)
        co1_ms = time_kernel(lambda: co_launch(True), reps)
        coissue = {"mfma_alone_tflops": round(co_flops[0] / (co0_ms * 1e-3) / 1e12, 1),
                   "mfma_beside_softmax_tflops": round(co_flops[0] / (co1_ms * 1e-3) / 1e12, 1),
                   "mfma_share_beside_softmax": round(co0_ms / co1_ms, 4)}

    # merge of all C states of a layer into the fp32 result, rotating over the layers' arenas
    dst_n = max(1, min(8, int(1.2e9 // (rows * (4 * D + 4))) + 1))
    dst_os = [torch.empty(B, Sq, H, D, dtype=torch.float32, device=dev) for _ in range(dst_n)]
    dst_ls = [torch.empty(B, Sq, H, 1, dtype=torch.float32, device=dev) for _ in range(dst_n)]

    def merge_layer(i):
        cache = layers[i % L_run].cache
        outs = [cache.arena_out[c] if c != diag else cache.diag_out for c in range(C)]
        lses = [cache.arena_lse[c] if c != diag else cache.diag_lse for c in range(C)]
        _hip.merge_states(outs, lses, dst_out=dst_os[i % dst_n], dst_lse=dst_ls[i % dst_n])

    k2_ms = time_kernel(Rotation(merge_layer, L_run * dst_n), reps)
    k2_bytes = rows * (C * (2 * D + 4) + (4 * D + 4))
    k2_gbs = k2_bytes / (k2_ms * 1e-3) / 1e9

    # the reference's own use of the merge: a running fp32 (out, lse [B,S,H,1]) updated in place with one bf16 block
    # state (utils.py:24-84 as called at core/attention.py:116,144,194,196,213), rotating over states and slots
    def update_running(i):
        cache = layers[i % L_run].cache
        c = (i // L_run) % C
        blk = (cache.arena_out[c], cache.arena_lse[c]) if c != diag else (cache.diag_out, cache.diag_lse)
        _hip.merge_states([dst_os[i % dst_n], blk[0]], [dst_ls[i % dst_n], blk[1]], dst_out=dst_os[i % dst_n], dst_lse=dst_ls[i % dst_n])

    k2u_ms = time_kernel(Rotation(update_running, L_run * C * dst_n), reps)
    k2u_bytes = rows * ((2 * D + 4) + 2 * (4 * D + 4))
    k2u_gbs = k2u_bytes / (k2u_ms * 1e-3) / 1e9
    k2_ws_mb = (L_run * C * state_bytes + dst_n * rows * (4 * D + 4)) / 1e6

    # cache store / load, over a rotation of cache slots of distinct layers and of source / destination tensors
    slots = [(layers[l].cache.arena_out[c], layers[l].cache.arena_lse[c]) for l in range(L_run) for c in range(C) if c != diag]
    n_slots = max(1, min(len(slots), int(1.5e9 // state_bytes) + 1))
    k3s_ms = time_kernel(Rotation(lambda i: _hip.cache_store(dst_os[i % dst_n], dst_ls[i % dst_n], *slots[i % n_slots]),
                                  n_slots * dst_n), reps)
    k3s_gbs = rows * ((4 * D + 4) + (2 * D + 4)) / (k3s_ms * 1e-3) / 1e9
    k3c_ms = time_kernel(Rotation(lambda i: _hip.cache_store(*slots[i % n_slots], *slots[(i + n_slots // 2 + 1) % n_slots]),
                                  n_slots), reps)
    k3c_gbs = rows * 2 * (2 * D + 4) / (k3c_ms * 1e-3) / 1e9
    k3l_ms = time_kernel(Rotation(lambda i: _hip.cache_load(*slots[i % n_slots], dst_out=dst_os[i % dst_n],
                                                            dst_lse=dst_ls[i % dst_n]), n_slots * dst_n), reps)
    k3l_gbs = rows * ((2 * D + 4) + (4 * D + 4)) / (k3l_ms * 1e-3) / 1e9
    copy_ws_mb = (n_slots * state_bytes + dst_n * rows * (4 * D + 4)) / 1e6

    # the yardstick: what the memory system delivers to a read-only kernel with the merge's access pattern
    # (the bf16 halves of C cache slots, rotating over the layers)
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    probe_bytes = rows * D * 2 // 256 * 256

    def probe(i):
        cache = layers[i % L_run].cache
        bench_probes.hbm_read_probe([cache.arena_out[c] for c in range(C)], sink)

    kr_ms = time_kernel(Rotation(probe, L_run), reps)
    kr_gbs = C * probe_bytes / (kr_ms * 1e-3) / 1e9

    # what launches of these grids cost before they move a byte: an empty kernel of the merge's grid (16 units of 128
    # elements per 256-thread workgroup and pass; two passes for 6 and more states at D = 128 and for launches of 2^20
    # units and more at D = 64) and of the flat copy's (8 KB per 512-thread workgroup)
    units = rows * D // 128
    merge_passes = 2 if ((D == 128 and C >= 6) or (D == 64 and units >= (1 << 20))) else 1
    merge_wgs = -(-units // (16 * merge_passes))
    copy_wgs = -(-(rows * (2 * D + 4)) // 8192)
    floor_merge_ms = time_kernel(lambda: bench_probes.empty_launch(merge_wgs, 256), reps)
    floor_copy_ms = time_kernel(lambda: bench_probes.empty_launch(copy_wgs, 512), reps)
    launch_floor = {"merge_grid": [merge_wgs, 256], "merge_grid_us": round(floor_merge_ms * 1e3, 2),
                    "copy_grid": [copy_wgs, 512], "copy_grid_us": round(floor_copy_ms * 1e3, 2),
                    "what": "an empty kernel of the same grid, launched back to back: the part of a short launch that is not bandwidth"}

    traffic = load_traffic(name)   # per launch shape: the same whatever reuse fraction drew the mask
    # counter bytes of exactly the launch shape that is timed next to them, or nothing
    k1_traffic = traffic.get("attn_fwd", {}).get(str(n_typ)) if isinstance(traffic.get("attn_fwd"), dict) else None
    k2_traffic = traffic.get("merge_states", {}).get(str(C)) if isinstance(traffic.get("merge_states"), dict) else None
    frac = k1_tflops / PEAK_BF16_TFLOPS
    roofline = {"kernel": "attn_fwd_kernel<%d>" % D, "bound": "mfma", "achieved": round(k1_tflops, 1),
                "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(frac, 4),
                "traffic": k1_traffic, "launch_ms": round(k1_ms, 4), "flop_per_launch": k1_flops(n_typ),
                "chunks_per_launch": n_typ, "single_chunk_launch_tflops": round(k1s_tflops, 1),
                "single_chunk_launch_ms": round(k1s_ms, 4),
                "q_prescaled_launch_tflops": round(k1p_tflops, 1), "q_prescaled_launch_ms": round(k1p_ms, 4),
                "fp16_launch_tflops": round(k1h_tflops, 1), "fp16_launch_ms": round(k1h_ms, 4)}
    if clock:
        # the part is power-limited under this kernel: what the kernel reaches of the peak AT THE CLOCK IT RUNS AT
        roofline["clock_mhz_under_load"] = clock
        roofline["frac_at_clock"] = round(frac * NOMINAL_CLOCK_MHZ / clock, 4)
    if watts:
        roofline["power_w_under_load"] = watts
        roofline["power_cap_w"] = power_cap_w()
    if mfma_probe:
        roofline["mfma_probe_tflops"] = mfma_probe["tflops"]
        roofline["mfma_probe_clock_mhz"] = mfma_probe["clock_mhz_under_load"]
        if mfma_probe["power_w_under_load"]:
            roofline["mfma_probe_power_w"] = mfma_probe["power_w_under_load"]
        roofline["frac_of_mfma_probe"] = round(k1_tflops / mfma_probe["tflops"], 4)
    if coissue:
        roofline["coissue_probe"] = coissue
        roofline["frac_of_coissue_ceiling"] = round(k1_tflops / coissue["mfma_beside_softmax_tflops"], 4)
    roofline_merge = {"kernel": "merge_states_kernel<%d>" % D, "bound": "hbm", "achieved": round(k2_gbs, 1),
                      "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(k2_gbs / PEAK_HBM_GBS, 4),
                      "traffic": k2_traffic, "launch_us": round(k2_ms * 1e3, 2), "bytes_per_launch": k2_bytes,
                      "states": C, "working_set_mb": round(k2_ws_mb, 0),
                      "read_probe_gbs": round(kr_gbs, 1), "frac_of_read_probe": round(k2_gbs / kr_gbs, 4),
                      "running_update": {"what": "fp32 running state updated in place with one bf16 block (update_out_and_lse as the reference calls it)",
                                         "gbs": round(k2u_gbs, 1), "frac": round(k2u_gbs / PEAK_HBM_GBS, 4),
                                         "launch_us": round(k2u_ms * 1e3, 2), "bytes_per_launch": k2u_bytes}}
    cache_gbs = {"store_fp32_to_slot": round(k3s_gbs, 1), "store_bf16_to_slot": round(k3c_gbs, 1),
                 "load_slot_to_fp32": round(k3l_gbs, 1), "peak": PEAK_HBM_GBS,
                 "frac_store_bf16": round(k3c_gbs / PEAK_HBM_GBS, 4), "frac_load": round(k3l_gbs / PEAK_HBM_GBS, 4),
                 "working_set_mb": round(copy_ws_mb, 0), "slots_rotated": n_slots}
    cfg_rec = {"workload": label, "B": B, "H": H, "D": D, "Sq": Sq, "kv_chunks": C, "Sk": lens[0],
               "mask": f"Bernoulli({p}) seed 0 over {T}x{L}x{C}, diag {diag}", "layers_instantiated": L_run,
               "mean_chunks_computed_per_call": round(mean_computed, 3),
               "schedule_mean_chunks_computed_per_call": round(population_mean, 3)}
    layer_tflops = flops_per_chunk * mean_computed / (ms_per_step * 1e-3) / 1e12

    if not main:
        rec = {"config": cfg_rec, "ms_per_layer": round(ms_per_step, 4), "steps": steps,
               "ms_per_layer_schedule_mean": round(schedule_mean_ms, 4),
               "layer_attn_tflops": round(layer_tflops, 1),
               "attn": {"frac": roofline["frac"], "tflops": roofline["achieved"], "chunks_per_launch": n_typ,
                        "launch_ms": roofline["launch_ms"], "single_chunk_frac": round(k1s_tflops / PEAK_BF16_TFLOPS, 4),
                        "q_prescaled_frac": round(k1p_tflops / PEAK_BF16_TFLOPS, 4),
                        "fp16_frac": round(k1h_tflops / PEAK_BF16_TFLOPS, 4), "traffic": k1_traffic,
                        "coissue_probe": coissue,
                        "frac_of_coissue_ceiling": roofline.get("frac_of_coissue_ceiling")},
               "merge": {"frac": roofline_merge["frac"], "gbs": roofline_merge["achieved"], "states": C,
                         "launch_us": roofline_merge["launch_us"], "read_probe_gbs": roofline_merge["read_probe_gbs"],
                         "traffic": k2_traffic},
               "cache_gbs": {"store_bf16_to_slot": cache_gbs["store_bf16_to_slot"], "load_slot_to_fp32": cache_gbs["load_slot_to_fp32"],
                             "store_bf16_launch_us": round(k3c_ms * 1e3, 2), "load_launch_us": round(k3l_ms * 1e3, 2)},
               "launch_floor": launch_floor}
    else:
        # producer step of the callers: RMSNorm + interleaved RoPE of K over the whole KV sequence, read in
        # place from a fused QKV projection ("B L (K H D)"), written as the [B,S,H,D] bf16 the attention reads
        S_all = int(sum(lens))
        qkv = torch.randn(B, S_all, 3, H, D, device=dev, dtype=torch.bfloat16)
        ang = torch.rand(S_all, D // 2, device=dev) * 6.28
        p_cos = ang.cos().repeat_interleave(2, -1).contiguous()
        p_sin = ang.sin().repeat_interleave(2, -1).contiguous()
        p_w = torch.ones(D, device=dev)
        p_out = torch.empty(B, S_all, H, D, dtype=torch.bfloat16, device=dev)
        kp_ms = time_kernel(lambda: _hip.qk_norm_rope(qkv[:, :, 1], norm=_hip.DT_NORM_RMS, weight=p_w, rope=_hip.DT_ROPE_INTERLEAVED,
                                                      cos=p_cos, sin=p_sin, out=p_out), reps, warm=40)
        kp_bytes = B * S_all * H * D * 4 + S_all * D * 8
        kp_gbs = kp_bytes / (kp_ms * 1e-3) / 1e9
        del qkv, ang, p_cos, p_sin, p_out
        # the variable-length entry (HunyuanVideo's real one: two segments per sample, the valid tokens and the
        # padded text tokens, core/attention.py:239-419) on the same schedule rows: every scheduled chunk runs
        # once per segment inside one launch
        pad_rows = 64
        cu = [0, Sq - pad_rows, Sq]
        # the boundaries are int32 tensors ON THE GPU, as the model makes them (hunyuan_transformer.py:789-792) and as
        # they travel with K/V round the ring (core/attention.py:307-311); max_seqlen = the sample's length (:783-784)
        cu_kv_ts = [torch.tensor([0, n - pad_rows, n], dtype=torch.int32, device=dev) for n in lens]
        group.set_kv_chunks(ks, vs, cu_seqlens_kv=cu_kv_ts)
        q3, k3, v3 = q.view(B * Sq, H, D), ks[rank].view(B * lens[rank], H, D), vs[rank].view(B * lens[rank], H, D)
        cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
        cu_kv_t = cu_kv_ts[rank]
        n_var = 1 if kernels_only else min(24, len(timed))

        def run_varlen(t, l):
            update_timestep(t)
            return layers[l].varlen_attn(q3, k3, v3, cu_t, cu_kv_t, Sq, max(lens))

        for t, l in timed[:2]:
            run_varlen(t, l)
        torch.cuda.synchronize()
        t0v = time.perf_counter()
        for t, l in timed[:n_var]:
            run_varlen(t, l)
        torch.cuda.synchronize()
        var_ms = 1e3 * (time.perf_counter() - t0v) / n_var
        var_chunks = float(np.mean(n_comp[:n_var]))
        var_flops = 4.0 * H * D * ((Sq - pad_rows) * (Sk_mean - pad_rows) + pad_rows * pad_rows) * B * var_chunks
        group.set_kv_chunks(ks, vs)
        # profiling mode: the relative-L1 sums of two fp32 outputs (record_out_redundancy, utils.py:202-267)
        sums = torch.zeros(4, dtype=torch.float64, device=dev)
        kl_ms = time_kernel(Rotation(lambda i: _hip.rel_l1_sums(dst_os[i % dst_n], dst_os[(i + 1) % dst_n], sums), dst_n), reps)
        kl_gbs = 2 * rows * D * 4 / (kl_ms * 1e-3) / 1e9
        dmask = torch.from_numpy(mask).to(dev)
        k4_ms = time_kernel(lambda: _hip.build_schedule_table(dmask, diag), reps)
        # a plain copy of known size: the yardstick the profiler's FETCH_SIZE / WRITE_SIZE counters are scaled by
        ref_src = torch.empty(1 << 28, dtype=torch.float32, device=dev)   # 1 GiB
        ref_dst = torch.empty_like(ref_src)
        copy_ms = time_kernel(lambda: ref_dst.copy_(ref_src), max(3, reps // 4))
        copy_gbs = 2 * ref_src.numel() * 4 / (copy_ms * 1e-3) / 1e9
        del ref_src, ref_dst
        rec = {
            "metric": "ms/layer", "value": round(ms_per_step, 4), "unit": "ms", "n_gpus": 1,
            "steps": steps, "warmup": warmup, "ms_per_step": round(ms_per_step, 4),
            "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": cfg_rec,
            "ms_per_layer_schedule_mean": round(schedule_mean_ms, 4),
            "ms_by_chunks_computed": {str(k): round(float(np.mean(v)), 4) for k, v in sorted(per_count.items())},
            "layer_attn_tflops": round(layer_tflops, 1),
            "roofline": roofline, "roofline_merge": roofline_merge, "cache_gbs": cache_gbs, "launch_floor": launch_floor,
            "producer": {"kernel": "qk_norm_rope_kernel<%d>" % D, "bound": "hbm", "achieved": round(kp_gbs, 1),
                         "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(kp_gbs / PEAK_HBM_GBS, 4),
                         "launch_us": round(kp_ms * 1e3, 2), "bytes_per_launch": kp_bytes, "tokens": S_all,
                         "what": "RMSNorm + interleaved RoPE of K over the whole KV sequence, strided read from a fused QKV tensor"},
            "varlen": {"what": f"proAttention.varlen_attn, two segments per sample ({Sq - pad_rows} + {pad_rows} query rows; "
                               f"{lens[0] - pad_rows} + {pad_rows} keys per chunk), same schedule rows",
                       "cu_seqlens": "device (int32 tensors on the GPU, read by the kernel; no host sync per call)",
                       "ms_per_layer": round(var_ms, 4), "calls": n_var, "mean_chunks_computed_per_call": round(var_chunks, 3),
                       "layer_attn_tflops": round(var_flops / (var_ms * 1e-3) / 1e12, 1)},
            "rel_l1": {"kernel": "rel_l1_sums_kernel", "bound": "hbm", "achieved": round(kl_gbs, 1), "peak": PEAK_HBM_GBS,
                       "unit": "GB/s", "frac": round(kl_gbs / PEAK_HBM_GBS, 4), "launch_us": round(kl_ms * 1e3, 2),
                       "bytes_per_launch": 2 * rows * D * 4},
            "schedule_builder_us": round(k4_ms * 1e3, 2),
            "plain_copy_1GiB_gbs": round(copy_gbs, 1),
        }
    # release this workload's memory before the next one
    for a in layers:
        a.cache.release()
    del layers, q, ks, vs, table, st_outs, st_lses, dst_os, dst_ls, slots
    group.set_kv_chunks([None] * C, [None] * C)
    rmod.destroy_redundancy_map()
    parallel_state.destroy_local_groups()
    update_timestep(0)
    torch.cuda.empty_cache()
    rec["_mean_computed"] = mean_computed
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=120)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="hunyuanvideo", choices=list(WORKLOADS))
    ap.add_argument("--layers", type=int, default=None, help="layers to instantiate (default: all of the model)")
    ap.add_argument("--reuse", type=float, default=None, help="override the mask's reuse probability")
    ap.add_argument("--kernel-reps", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true", help="skip the compact records of the other configurations")
    ap.add_argument("--schedule", default="mask", choices=["mask", "stride"],
                    help="mask: the seeded Bernoulli reuse mask (the headline metric); stride: the reference's own stride "
                         "schedule from the HunyuanVideo redundancy map it ships (a separate, shorter report)")
    ap.add_argument("--item-model", action="store_true",
                    help="a separate report: the attention kernel's time per key tile and per work item, fitted from launches "
                         "that exactly fill the chip (both head dimensions)")
    ap.add_argument("--kernels-only", action="store_true",
                    help="run only the per-kernel roofline launches (short; for rocprofv3 counter passes)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one sequence-parallel rank's share on ONE GPU; --gpus > 1 is not part of this build",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)

    from ditango_amd import _hip
    from ditango_amd.logger import init_logger
    import logging
    init_logger("bench")
    for h in logging.getLogger("ditango_amd").handlers:     # stdout carries the one JSON line only
        if isinstance(h, logging.StreamHandler) and not isinstance(h, logging.FileHandler):
            h.setStream(sys.stderr)
    _hip.load_library()
    torch.cuda.set_device(0)
    global PROFILING
    PROFILING = args.kernels_only

    if args.item_model:
        return bench_item_model(args)
    if args.schedule == "stride":
        return bench_stride_schedule(args)
    result = run_workload(args.workload, args, args.steps, args.warmup, main=True, reuse=args.reuse,
                          kernels_only=args.kernels_only)
    mean_computed = result.pop("_mean_computed")
    if not args.kernels_only and not args.no_other_configs and args.workload == "hunyuanvideo" and args.reuse is None:
        others = {}
        for name, reuse in (("cogvideox", None), ("stepvideo", None), ("sweep", 0.5), ("sweep", 0.9)):
            steps = 40 if name != "sweep" else 6
            rec = run_workload(name, args, steps, 4 if name != "sweep" else 2, main=False, reuse=reuse)
            rec.pop("_mean_computed")
            others[name if name != "sweep" else f"sweep_reuse_{reuse}"] = rec
        # the reference's own mode: the stride schedule of the redundancy map it ships, every call timed
        others["stride_schedule"] = stride_schedule_record(args.layers or 6)
        result["other_configs"] = others
    if not args.no_cpu_baseline and not args.kernels_only:
        label, B, H, D, Sq, lens, T, L, p, diag, norm = WORKLOADS[args.workload]
        result["cpu_baseline"] = cpu_baseline(B, H, D, Sq, lens, mean_computed, len(lens), norm)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
