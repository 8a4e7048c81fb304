#!/usr/bin/env python3
"""Benchmark of the cached block attention hot path on ONE MI355X.

A "step" is one ``proAttention.attn`` call (one transformer layer's attention at one
diffusion step) at the HunyuanVideo per-rank shape: local query shard of 14882 tokens,
KV = 8 chunks of 14882 tokens, H=24, D=128, bf16, under the seeded Bernoulli(0.6) reuse mask
over 50 steps x 60 layers.  Inputs are resident in HBM before the timed region.

Prints ONE JSON line: ms per layer call plus
  * ``roofline``        the fresh-chunk attention kernel against the bf16 dense MFMA peak,
  * ``roofline_merge``  the fused LSE-merge kernel against the HBM peak,
  * ``cache_gbs``       cache store / load copies against the HBM peak,
  * ``cpu_baseline``    the torch-math oracle timed on this box's host cores on a bounded sample.
"""
import argparse
import json
import math
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

WORKLOADS = {
    # name: (label, B, H, D, Sq, chunk lengths, T, L, reuse probability, diag, qk norm)
    "hunyuanvideo": ("HunyuanVideo per-rank share (configs[2])", 1, 24, 128, 14882, [14882] * 8, 50, 60, 0.6, 0, "rms"),
    "cogvideox": ("CogVideoX-5B per-rank share (configs[1])", 1, 48, 64, 2222, [2222] * 8, 50, 42, 0.5, 0, "layer"),
    "stepvideo": ("Step-Video-T2V per-rank share (configs[3])", 1, 48, 128, 6851, [6851] * 8, 50, 48, 0.75, 0, None),
    "sweep": ("reuse sweep at HunyuanVideo scale (configs[4])", 1, 24, 128, 119056, [3721] * 16 + [3720] * 16, 1, 60, 0.5, -1, "rms"),
}


def make_inputs(B, H, D, Sq, lens, norm, device, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed)

    def draw(n, normalise):
        x = torch.randn(B, n, H, D, generator=g)
        if normalise == "rms":
            x = x / x.pow(2).mean(-1, keepdim=True).sqrt()
        elif normalise == "layer":
            x = torch.nn.functional.layer_norm(x, (D,))
        return x.bfloat16()

    q = draw(Sq, norm).to(device)
    ks = [draw(n, norm).to(device) for n in lens]
    vs = [draw(n, None).to(device) for n in lens]
    return q, ks, vs


def time_kernel(fn, reps, warm=3):
    """Average duration in ms of ``fn`` over ``reps`` launches (HIP events on the launch stream)."""
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
    if total < 40.0:  # short kernels: time at least 40 ms of them, so that clock ramps average out
        more = int(reps * 40.0 / max(total, 1e-3)) + 1
        e0.record()
        for _ in range(more):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / more
    return total / reps


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


def bench_stride_schedule(args):
    """One full pass of the reference's stride schedule: 50 steps x ``--layers`` layers (default 12) of
    ``proAttention.attn`` at the HunyuanVideo per-rank shape as ring rank 0 of 8, with the divider map
    generated from the redundancy map the reference ships for HunyuanVideo (percentiles [0,40,90],
    dividers [8,4,2,1], configs/hunyuanvideo/config.yaml).  Every call is timed, the full-stride
    steps included."""
    from ditango_amd.core import config, parallel_state, redundancy_map as rmod
    from ditango_amd.core.attention import proAttention
    from ditango_amd.utils import update_timestep
    label, B, H, D, Sq, lens, T, L, _, _, norm = WORKLOADS["hunyuanvideo"]
    N, rank = len(lens), 0
    L_run = min(L, args.layers or 12)
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    parallel_state.init_local_groups(N, rank)
    cfg = config.init_config(None, num_inference_steps=T, num_layers=L, stride_percentiles=[0, 40, 90],
                             stride_dividers=[8, 4, 2, 1])
    rmod.destroy_redundancy_map()
    rm = rmod.init_redundancy_map(cfg, redun_map_path=os.path.join(ROOT, "tests", "golden", "redundancy_map_50_60.pt"),
                                  quiet=True)
    q, ks, vs = make_inputs(B, H, D, Sq, lens, norm, dev)
    group = parallel_state.get_usp_group()
    group.set_kv_chunks(ks, vs)
    layers = [proAttention(l, group) for l in range(L_run)]
    computed = 0
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for t in range(T):
        update_timestep(t)
        for l in range(L_run):
            layers[l].attn(q, ks[rank], vs[rank])
            computed += len(layers[l].last_plan.computed)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    calls = T * L_run
    flops = 4.0 * B * H * Sq * lens[0] * D * computed
    print(json.dumps({
        "metric": "ms/layer", "value": round(1e3 * elapsed / calls, 4), "unit": "ms", "n_gpus": 1, "steps": calls, "warmup": 0,
        "ms_per_step": round(1e3 * elapsed / calls, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": label + ", stride schedule of the shipped redundancy map, ring rank 0 of 8", "B": B, "H": H,
                   "D": D, "Sq": Sq, "kv_chunks": N, "Sk": lens[0], "layers_instantiated": L_run, "steps_per_layer": T,
                   "mean_chunks_computed_per_call": round(computed / calls, 3)},
        "layer_attn_tflops": round(flops / elapsed / 1e12, 1),
    }), flush=True)


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
    ap.add_argument("--schedule", default="mask", choices=["mask", "stride"],
                    help="mask: the seeded Bernoulli reuse mask (the headline metric); stride: the reference's own stride "
                         "schedule from the HunyuanVideo redundancy map it ships (a separate, shorter report)")
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
    from ditango_amd.core import config, parallel_state, redundancy_map as rmod
    from ditango_amd.core.attention import proAttention
    from ditango_amd.utils import update_timestep
    _hip.load_library()

    if args.schedule == "stride":
        return bench_stride_schedule(args)
    label, B, H, D, Sq, lens, T, L, p, diag, norm = WORKLOADS[args.workload]
    if args.reuse is not None:
        p = args.reuse
    C = len(lens)
    L_run = min(L, args.layers) if args.layers else L
    if args.workload == "sweep":
        L_run = min(L_run, 2)   # 32 cached states of 743 MB per layer
        T = 2                   # step 0 fills the cache, step 1 is measured
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
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

    calls = [(t, l) for t in range(1, T) for l in range(L_run)]
    need = args.warmup + args.steps
    seq = [calls[i % len(calls)] for i in range(need)]

    def run(t, l):
        update_timestep(t)
        return layers[l].attn(q, ks[rank], vs[rank])

    planned = seq[args.warmup:]   # the calls the default run times (also fixes the typical launch below)
    if args.kernels_only:
        args.warmup, args.steps = 0, 1
        seq = seq[:1]
    for t, l in seq[:args.warmup]:
        run(t, l)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for t, l in seq[args.warmup:]:
        run(t, l)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = 1e3 * elapsed / args.steps
    n_comp = [int(rm.sched_counts_host[t, l, 0]) for t, l in planned]
    mean_computed = float(np.mean(n_comp))
    Sk_mean = float(np.mean(lens))
    flops_per_chunk = 4.0 * B * H * Sq * Sk_mean * D
    rows = B * Sq * H

    # ---- per-kernel rooflines, measured live with HIP events on the launch stream ----------
    reps = args.kernel_reps
    out_s = torch.empty(B, Sq, H, D, dtype=torch.bfloat16, device=dev)
    lse_s = torch.empty(B, H, Sq, dtype=torch.float32, device=dev)
    # the dominant kernel in its typical launch: as many single-chunk states as a layer call
    # computes on average (rounded), written into cache slots, one launch
    n_typ = max(1, min(C, int(round(mean_computed))))
    table = _hip.ChunkTable(ks, vs)
    typ_jobs = [[c] for c in range(n_typ)]
    typ_outs = [torch.empty_like(out_s) for _ in range(n_typ)]
    typ_lses = [torch.empty_like(lse_s) for _ in range(n_typ)]
    k1_ws = _hip.attn_workspace(dev)   # the launch as proAttention makes it: with the tail-balancing workspace
    k1_ms = time_kernel(lambda: _hip.attn_jobs_fwd(q, table, typ_jobs, typ_outs, typ_lses, workspace=k1_ws), reps)
    k1_flops = sum(4.0 * B * H * Sq * lens[c] * D for c in range(n_typ))
    k1_tflops = k1_flops / (k1_ms * 1e-3) / 1e12
    k1s_ms = time_kernel(lambda: _hip.attn_jobs_fwd(q, table, [[0]], [out_s], [lse_s], workspace=k1_ws), reps)
    k1s_tflops = 4.0 * B * H * Sq * lens[0] * D / (k1s_ms * 1e-3) / 1e12
    # the same typical launch in the opt-in mode of a caller that folds softmax_scale * log2(e) into q
    # (reported beside the drop-in figure, never in place of it)
    q_folded = (q.float() * (D ** -0.5 * math.log2(math.e))).to(torch.bfloat16)
    k1p_ms = time_kernel(lambda: _hip.attn_jobs_fwd(q_folded, table, typ_jobs, typ_outs, typ_lses, workspace=k1_ws,
                                                    q_prescaled=True), reps)
    k1p_tflops = k1_flops / (k1p_ms * 1e-3) / 1e12
    del typ_outs, typ_lses, q_folded

    cache0 = layers[0].cache
    m_outs = [cache0.arena_out[c] if c != diag else cache0.diag_out for c in range(C)]
    m_lses = [cache0.arena_lse[c] if c != diag else cache0.diag_lse for c in range(C)]
    dst_o = torch.empty(B, Sq, H, D, dtype=torch.float32, device=dev)
    dst_l = torch.empty(B, Sq, H, 1, dtype=torch.float32, device=dev)
    k2_ms = time_kernel(lambda: _hip.merge_states(m_outs, m_lses, dst_out=dst_o, dst_lse=dst_l), reps)
    k2_bytes = rows * (C * (2 * D + 4) + (4 * D + 4))
    k2_gbs = k2_bytes / (k2_ms * 1e-3) / 1e9

    k3s_ms = time_kernel(lambda: _hip.cache_store(dst_o, dst_l, out_s, lse_s), reps)
    k3s_gbs = rows * ((4 * D + 4) + (2 * D + 4)) / (k3s_ms * 1e-3) / 1e9
    slot2_o, slot2_l = torch.empty_like(out_s), torch.empty_like(lse_s)
    k3c_ms = time_kernel(lambda: _hip.cache_store(out_s, lse_s, slot2_o, slot2_l), reps)
    k3c_gbs = rows * 2 * (2 * D + 4) / (k3c_ms * 1e-3) / 1e9
    k3l_ms = time_kernel(lambda: _hip.cache_load(out_s, lse_s, torch.float32, True), reps)
    k3l_gbs = rows * ((2 * D + 4) + (4 * D + 4)) / (k3l_ms * 1e-3) / 1e9

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

    dmask = torch.from_numpy(mask).to(dev)
    k4_ms = time_kernel(lambda: _hip.build_schedule_table(dmask, diag), reps)
    # a plain copy of known size: the yardstick the profiler's FETCH_SIZE / WRITE_SIZE counters are scaled by
    ref_src = torch.empty(1 << 28, dtype=torch.float32, device=dev)   # 1 GiB
    ref_dst = torch.empty_like(ref_src)
    copy_ms = time_kernel(lambda: ref_dst.copy_(ref_src), max(3, reps // 4))
    copy_gbs = 2 * ref_src.numel() * 4 / (copy_ms * 1e-3) / 1e9
    del ref_src, ref_dst

    # HBM bytes per launch measured offline with rocprofv3 counters (FETCH_SIZE + WRITE_SIZE),
    # committed as text under profiles/; only meaningful for the default workload
    traffic = {}
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic_hunyuanvideo.json")
    if args.workload == "hunyuanvideo" and args.reuse is None and os.path.exists(tpath):
        with open(tpath) as f:
            traffic = json.load(f).get("bytes_per_launch", {})

    result = {
        "metric": "ms/layer", "value": round(ms_per_step, 4), "unit": "ms", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": label, "B": B, "H": H, "D": D, "Sq": Sq, "kv_chunks": C, "Sk": lens[0],
                   "mask": f"Bernoulli({p}) seed 0 over {T}x{L}x{C}, diag {diag}", "layers_instantiated": L_run,
                   "mean_chunks_computed_per_call": round(mean_computed, 3)},
        "layer_attn_tflops": round(flops_per_chunk * mean_computed / (ms_per_step * 1e-3) / 1e12, 1),
        "roofline": {"kernel": "attn_fwd_kernel<%d>" % D, "bound": "mfma", "achieved": round(k1_tflops, 1),
                     "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(k1_tflops / PEAK_BF16_TFLOPS, 4),
                     "traffic": traffic.get("attn_fwd"), "launch_ms": round(k1_ms, 4), "flop_per_launch": k1_flops,
                     "chunks_per_launch": n_typ, "single_chunk_launch_tflops": round(k1s_tflops, 1),
                     "single_chunk_launch_ms": round(k1s_ms, 4),
                     "q_prescaled_launch_tflops": round(k1p_tflops, 1), "q_prescaled_launch_ms": round(k1p_ms, 4)},
        "roofline_merge": {"kernel": "merge_states_kernel<%d>" % D, "bound": "hbm", "achieved": round(k2_gbs, 1),
                           "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(k2_gbs / PEAK_HBM_GBS, 4),
                           "traffic": traffic.get("merge_states"), "launch_us": round(k2_ms * 1e3, 2), "bytes_per_launch": k2_bytes,
                           "states": C},
        "cache_gbs": {"store_fp32_to_slot": round(k3s_gbs, 1), "store_bf16_to_slot": round(k3c_gbs, 1),
                      "load_slot_to_fp32": round(k3l_gbs, 1), "peak": PEAK_HBM_GBS,
                      "frac_store_bf16": round(k3c_gbs / PEAK_HBM_GBS, 4), "frac_load": round(k3l_gbs / PEAK_HBM_GBS, 4)},
        "producer": {"kernel": "qk_norm_rope_kernel<%d>" % D, "bound": "hbm", "achieved": round(kp_gbs, 1),
                     "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(kp_gbs / PEAK_HBM_GBS, 4),
                     "launch_us": round(kp_ms * 1e3, 2), "bytes_per_launch": kp_bytes, "tokens": S_all,
                     "what": "RMSNorm + interleaved RoPE of K over the whole KV sequence, strided read from a fused QKV tensor"},
        "schedule_builder_us": round(k4_ms * 1e3, 2),
        "plain_copy_1GiB_gbs": round(copy_gbs, 1),
    }
    if not args.no_cpu_baseline and not args.kernels_only:
        result["cpu_baseline"] = cpu_baseline(B, H, D, Sq, lens, mean_computed, C, norm)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
