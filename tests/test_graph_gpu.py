"""A layer call's two launches (device-scheduled attention + N-way merge) captured in a HIP graph.

Possible because the entry points neither allocate nor synchronise and the schedule lives in device
memory: between replays only device buffers change (schedule row, K/V contents).  Every replay is
checked against the same two calls made eagerly, with eager work and synchronisations in between."""
import numpy as np
import pytest
import torch

from oracle import mask_schedule as ms

pytestmark = pytest.mark.gpu


def test_sched_attention_and_merge_replay_in_a_graph(hip):
    C, B, H, D, Sq, T, L = 6, 1, 3, 128, 150, 6, 1
    diag = 2
    g = torch.Generator().manual_seed(4)
    dev = "cuda"
    q = torch.randn(B, Sq, H, D, generator=g).bfloat16().to(dev)
    ks = [torch.randn(B, 90 + 7 * c, H, D, generator=g).bfloat16().to(dev) for c in range(C)]
    vs = [torch.randn(B, 90 + 7 * c, H, D, generator=g).bfloat16().to(dev) for c in range(C)]
    table = hip.ChunkTable(ks, vs)
    mask = ms.seeded_mask(T, L, C, 0.5, seed=9, diag=diag)
    comp, reu, cnt = hip.build_schedule_table(torch.from_numpy(mask).to(dev), diag)
    torch.cuda.synchronize()

    def buffers():
        return dict(arena_o=torch.zeros(C, B, Sq, H, D, dtype=torch.bfloat16, device=dev),
                    arena_l=torch.full((C, B, H, Sq), float("-inf"), device=dev),
                    diag_o=torch.zeros(B, Sq, H, D, dtype=torch.bfloat16, device=dev),
                    diag_l=torch.zeros(B, H, Sq, device=dev),
                    out=torch.zeros(B, Sq, H, D, device=dev), lse=torch.zeros(B, Sq, H, 1, device=dev),
                    ids=torch.zeros(C, dtype=torch.int32, device=dev), n=torch.zeros(1, dtype=torch.int32, device=dev))

    def layer_call(b):
        hip.attn_sched_fwd(q, table, b["ids"], b["n"], C, b["arena_o"], b["arena_l"], diag, b["diag_o"], b["diag_l"])
        outs = [b["arena_o"][c] if c != diag else b["diag_o"] for c in range(C)]
        lses = [b["arena_l"][c] if c != diag else b["diag_l"] for c in range(C)]
        hip.merge_states(outs, lses, dst_out=b["out"], dst_lse=b["lse"])

    eager, graphed = buffers(), buffers()
    # first call outside the capture: one-time kernel attribute set-up happens here
    for b in (eager, graphed):
        b["ids"].copy_(comp[0, 0]); b["n"].copy_(cnt[0, 0, 0:1])
        layer_call(b)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        layer_call(graphed)
    for t in range(1, T):
        # the inputs drift between steps, the schedule row changes: device-side updates only
        for k in ks:
            k.add_(0.01 * torch.randn_like(k))
        for b in (eager, graphed):
            b["ids"].copy_(comp[t, 0]); b["n"].copy_(cnt[t, 0, 0:1])
        layer_call(eager)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        n = int(cnt[t, 0, 0])
        print(f"replay t={t}: computes {comp[t, 0, :n].tolist()}", flush=True)
        assert torch.equal(graphed["out"], eager["out"]) and torch.equal(graphed["lse"], eager["lse"]), f"replay {t}"
        assert torch.equal(graphed["arena_o"], eager["arena_o"]) and torch.equal(graphed["arena_l"], eager["arena_l"])
    assert np.array_equal(comp.cpu().numpy(), ms.build_schedule_table(mask, diag)[0])


def test_varlen_launch_with_device_boundaries_replays_in_a_graph(hip):
    """The variable-length launch with its cu_seqlens in device memory, captured once and replayed while the
    BOUNDARIES (and K/V) change on the device: every replay equals the eager launch on the same boundaries,
    which a launch that had read them on the host at capture time could not do."""
    B, H, D, total, lens = 1, 4, 128, 700, [500, 420]
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(8)
    q = torch.randn(B, total, H, D, generator=g, device=dev).bfloat16()
    ks = [torch.randn(B, n, H, D, generator=g, device=dev).bfloat16() for n in lens]
    vs = [torch.randn(B, n, H, D, generator=g, device=dev).bfloat16() for n in lens]
    table = hip.ChunkTable(ks, vs)
    cu_q = torch.tensor([0, 600, 700], dtype=torch.int32, device=dev)
    cu_k = [torch.tensor([0, 400, 500], dtype=torch.int32, device=dev), torch.tensor([0, 300, 420], dtype=torch.int32, device=dev)]
    seg = hip.DeviceSegments(cu_q, cu_k, total)
    jobs, job_segs = [[0, 1], [0, 1]], [0, 1]

    def buffers():
        return dict(o=torch.zeros(B, total, H, D, dtype=torch.bfloat16, device=dev), l=torch.zeros(B, H, total, device=dev))

    def call(b):
        hip.attn_jobs_fwd(q, table, jobs, [b["o"]] * 2, [b["l"]] * 2, dev_segments=seg, job_segments=job_segs)

    eager, graphed = buffers(), buffers()
    call(graphed)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(graphed)
    splits = [(600, 400, 300), (512, 100, 420), (64, 500, 0), (700, 250, 250), (333, 1, 419)]
    seen = []
    for step, (sq, s0, s1) in enumerate(splits):
        cu_q.copy_(torch.tensor([0, sq, total], dtype=torch.int32))
        cu_k[0].copy_(torch.tensor([0, s0, lens[0]], dtype=torch.int32))
        cu_k[1].copy_(torch.tensor([0, s1, lens[1]], dtype=torch.int32))
        for k in ks + vs:
            k.add_(0.01 * torch.randn_like(k))
        call(eager)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(graphed["o"], eager["o"]) and torch.equal(graphed["l"], eager["l"]), f"replay {step}"
        seen.append(graphed["o"].clone())
    assert not torch.equal(seen[0], seen[1])


def test_noalloc_attention_replays_in_a_graph(hip):
    """The allocation-free entry point under capture: the attention launch (with its tail split inside the
    library's own scratch array and the fold kernel behind it) plus the merge, replayed four times
    while K/V drift, against the same launches made eagerly through the workspace entry point."""
    B, H, D, Sq, lens = 1, 24, 128, 3000, [2000, 1500]        # 2 x 288 work items: a tail of 64 is split
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(21)
    q = torch.randn(B, Sq, H, D, generator=g, device=dev).bfloat16()
    ks = [torch.randn(B, n, H, D, generator=g, device=dev).bfloat16() for n in lens]
    vs = [torch.randn(B, n, H, D, generator=g, device=dev).bfloat16() for n in lens]
    table = hip.ChunkTable(ks, vs)
    jobs = [[0], [1]]
    ws = torch.empty(hip.DT_NOALLOC_TAIL_SLOTS * (256 * 128 * 2 + 256 * 4), dtype=torch.uint8, device=dev)

    def buffers():
        return dict(o=[torch.zeros(B, Sq, H, D, dtype=torch.bfloat16, device=dev) for _ in jobs],
                    l=[torch.zeros(B, H, Sq, device=dev) for _ in jobs],
                    out=torch.zeros(B, Sq, H, D, device=dev), lse=torch.zeros(B, Sq, H, 1, device=dev))

    def call(b, **how):
        hip.attn_jobs_fwd(q, table, jobs, b["o"], b["l"], **how)
        hip.merge_states(b["o"], b["l"], dst_out=b["out"], dst_lse=b["lse"])

    eager, graphed, plain = buffers(), buffers(), buffers()
    call(graphed, no_alloc=True)            # outside the capture: the scratch address is looked up here
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(graphed, no_alloc=True)
    for step in range(4):
        for k in ks + vs:
            k.add_(0.01 * torch.randn_like(k))
        call(eager, workspace=ws)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(graphed["out"], eager["out"]) and torch.equal(graphed["lse"], eager["lse"]), f"replay {step}"
        assert all(torch.equal(a, b) for a, b in zip(graphed["o"], eager["o"]))
    call(plain)
    torch.cuda.synchronize()
    assert any(not torch.equal(a, b) for a, b in zip(graphed["o"], plain["o"])), "the tail was expected to be split"
