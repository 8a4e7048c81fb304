"""The variable-length entry (HunyuanVideo): packed [total,H,D] inputs, segment i of the queries
attends to segment i of every KV chunk; segment boundaries of a chunk travel with the chunk."""
import pytest
import torch

from oracle import attention_math as om
from oracle.state_machine import RingOracle, strides_from_dividers

pytestmark = pytest.mark.gpu
OUT_TOL, LSE_TOL = 2e-2, 1e-3


@pytest.fixture
def env(hip):
    from ditango_amd.core import config, parallel_state, redundancy_map as rmod
    from ditango_amd import utils

    def make(N, rank, T, L):
        parallel_state.init_local_groups(N, rank)
        config.init_config(None, num_inference_steps=T, num_layers=L)
        rmod.destroy_redundancy_map()
        rmod._redundancy_map = rmod.RedundancyMap(config.get_config())
        return rmod.get_redundancy_map()

    yield make
    from ditango_amd.core import parallel_state, redundancy_map as rmod
    rmod.destroy_redundancy_map()
    parallel_state.destroy_local_groups()
    utils.update_timestep(0)


@pytest.mark.parametrize("D,cu_q,cu_k", [
    (128, [0, 300], [0, 333]),
    (128, [0, 257, 300], [0, 300, 333]),
    (64, [0, 100, 100, 290], [0, 64, 200, 333]),      # an empty query segment
    (128, [0, 10, 280], [0, 0, 333]),                 # a segment without keys
])
def test_segment_jobs_match_varlen_oracle(hip, D, cu_q, cu_k):
    H = 3
    g = torch.Generator().manual_seed(len(cu_q) + D)
    q = torch.randn(300, H, D, generator=g).bfloat16()
    k = torch.randn(333, H, D, generator=g).bfloat16()
    v = torch.randn(333, H, D, generator=g).bfloat16()
    ref_out, ref_lse = om.varlen_chunk_attention(q, k, v, cu_q, cu_k)
    dq, dk, dv = q.cuda()[None], k.cuda()[None], v.cuda()[None]
    out = torch.zeros(1, 300, H, D, dtype=torch.bfloat16, device="cuda")
    lse = torch.full((1, H, 300), float("-inf"), device="cuda")
    table = hip.ChunkTable([dk], [dv])
    nseg = len(cu_q) - 1
    hip.attn_jobs_fwd(dq, table, [[0]] * nseg, [out] * nseg, [lse] * nseg,
                      q_ranges=[(cu_q[i], cu_q[i + 1] - cu_q[i]) for i in range(nseg)],
                      kv_ranges=[[(cu_k[i], cu_k[i + 1] - cu_k[i])] for i in range(nseg)])
    torch.cuda.synchronize()
    assert (out[0].float().cpu() - ref_out).abs().max() <= OUT_TOL
    got, ref = lse[0].cpu(), ref_lse
    finite = torch.isfinite(ref)
    assert torch.equal(torch.isfinite(got), finite)
    assert (got[finite] - ref[finite]).abs().max() <= LSE_TOL


@pytest.mark.parametrize("D,cu_q,cu_k", [
    (128, [0, 300], [0, 333]),
    (128, [0, 257, 300], [0, 300, 333]),
    (64, [0, 100, 100, 290], [0, 64, 200, 333]),      # an empty query segment; rows 290.. in no segment
    (128, [0, 10, 280], [0, 0, 333]),                 # a segment without keys
    (64, [0, 40, 80, 120, 160, 200, 240, 250, 260, 270, 300], [0, 30, 60, 90, 120, 150, 180, 210, 240, 270, 333]),  # 10 segments
])
def test_segment_jobs_with_device_boundaries_equal_host_boundaries(hip, D, cu_q, cu_k):
    """dt_attn_varlen_jobs_fwd (cu_seqlens read by the kernel from device memory, flash_attn_varlen_func's calling
    convention) against dt_attn_seg_jobs_fwd (the same boundaries as host ranges): bit-identical states, and both
    within tolerance of the varlen oracle."""
    H = 3
    g = torch.Generator().manual_seed(len(cu_q) + D)
    q = torch.randn(300, H, D, generator=g).bfloat16()
    k = torch.randn(333, H, D, generator=g).bfloat16()
    v = torch.randn(333, H, D, generator=g).bfloat16()
    ref_out, ref_lse = om.varlen_chunk_attention(q, k, v, cu_q, cu_k)
    dq, dk, dv = q.cuda()[None], k.cuda()[None], v.cuda()[None]
    table = hip.ChunkTable([dk], [dv])
    nseg = len(cu_q) - 1
    res = []
    for on_device in (False, True):
        out = torch.zeros(1, 300, H, D, dtype=torch.bfloat16, device="cuda")
        lse = torch.full((1, H, 300), float("-inf"), device="cuda")
        if on_device:
            seg = hip.DeviceSegments(torch.tensor(cu_q, dtype=torch.int32, device="cuda"),
                                     [torch.tensor(cu_k, dtype=torch.int32, device="cuda")], max(b - a for a, b in zip(cu_q, cu_q[1:])))
            hip.attn_jobs_fwd(dq, table, [[0]] * nseg, [out] * nseg, [lse] * nseg, dev_segments=seg, job_segments=list(range(nseg)))
        else:
            hip.attn_jobs_fwd(dq, table, [[0]] * nseg, [out] * nseg, [lse] * nseg,
                              q_ranges=[(cu_q[i], cu_q[i + 1] - cu_q[i]) for i in range(nseg)],
                              kv_ranges=[[(cu_k[i], cu_k[i + 1] - cu_k[i])] for i in range(nseg)])
        torch.cuda.synchronize()
        res.append((out, lse))
    assert torch.equal(res[0][0], res[1][0]) and torch.equal(res[0][1], res[1][1])
    out, lse = res[1]
    assert (out[0].float().cpu() - ref_out).abs().max() <= OUT_TOL
    got, finite = lse[0].cpu(), torch.isfinite(ref_lse)
    assert torch.equal(torch.isfinite(got), finite) and (got[finite] - ref_lse[finite]).abs().max() <= LSE_TOL


def test_device_boundaries_are_clamped_and_checked(hip):
    """Nothing on the host reads device-resident boundaries, so the kernel clamps them to the rows and keys that
    exist: a list that overshoots both ends yields the full-range result, never a stray access.  What the host can
    check (dtype, placement, segment index, max_seqlen_q) is refused before any launch."""
    H, D = 2, 64
    g = torch.Generator().manual_seed(77)
    q = torch.randn(1, 200, H, D, generator=g).bfloat16().cuda()
    k = torch.randn(1, 150, H, D, generator=g).bfloat16().cuda()
    v = torch.randn(1, 150, H, D, generator=g).bfloat16().cuda()
    table = hip.ChunkTable([k], [v])
    full_o, full_l = hip.attn_chunk_fwd(q, k, v)
    out = torch.zeros_like(full_o)
    lse = torch.zeros_like(full_l)
    seg = hip.DeviceSegments(torch.tensor([-7, 100000], dtype=torch.int32, device="cuda"),
                             [torch.tensor([-3, 2 ** 30], dtype=torch.int32, device="cuda")], 200)
    hip.attn_jobs_fwd(q, table, [[0]], [out], [lse], dev_segments=seg, job_segments=[0])
    torch.cuda.synchronize()
    assert torch.equal(out, full_o) and torch.equal(lse, full_l)
    # decreasing boundaries: an empty segment (nothing written), no fault
    out.zero_()
    seg = hip.DeviceSegments(torch.tensor([150, 20], dtype=torch.int32, device="cuda"),
                             [torch.tensor([0, 150], dtype=torch.int32, device="cuda")], 200)
    hip.attn_jobs_fwd(q, table, [[0]], [out], [lse], dev_segments=seg, job_segments=[0])
    torch.cuda.synchronize()
    assert int(torch.count_nonzero(out)) == 0
    with pytest.raises(hip.DitangoHipError):
        hip.DeviceSegments(torch.tensor([0, 200], dtype=torch.int32), [torch.tensor([0, 150], dtype=torch.int32, device="cuda")], 200)
    with pytest.raises(hip.DitangoHipError):
        hip.DeviceSegments(torch.tensor([0, 200], dtype=torch.int64, device="cuda"), [None], 200)
    ok = hip.DeviceSegments(torch.tensor([0, 200], dtype=torch.int32, device="cuda"),
                            [torch.tensor([0, 150], dtype=torch.int32, device="cuda")], 200)
    with pytest.raises(hip.DitangoHipError):
        hip.attn_jobs_fwd(q, table, [[0]], [out], [lse], dev_segments=ok, job_segments=[1])      # segment index out of range
    with pytest.raises(hip.DitangoHipError):
        hip.DeviceSegments(ok.cu_q, ok.cu_kv, 0)


def test_zero_rows_from_a_device_index(hip):
    for first, n in ((0, 37), (20, 37), (37, 37), (-4, 10), (99, 10)):
        t = torch.ones(n, 3, 8, dtype=torch.float32, device="cuda")
        hip.zero_rows_from(t, torch.tensor([first], dtype=torch.int32, device="cuda"))
        torch.cuda.synchronize()
        lo = min(max(first, 0), n)
        assert bool((t[:lo] == 1).all()) and bool((t[lo:] == 0).all()), (first, n)


def test_single_segment_reduces_to_the_dense_path(env, hip):
    from ditango_amd.core.attention import proAttention
    from ditango_amd.core.parallel_state import get_usp_group
    N, S, H, D = 2, 150, 2, 128
    env(N, 0, 3, 1)
    g = torch.Generator().manual_seed(1)
    q = torch.randn(S, H, D, generator=g).bfloat16().cuda()
    ks = [torch.randn(S, H, D, generator=g).bfloat16().cuda() for _ in range(N)]
    vs = [torch.randn(S, H, D, generator=g).bfloat16().cuda() for _ in range(N)]
    group = get_usp_group()
    cu = torch.tensor([0, S], dtype=torch.int32)
    group.set_kv_chunks(ks, vs, cu_seqlens_kv=[cu] * N)
    a = proAttention(0, group).varlen_attn(q, ks[0], vs[0], cu, cu, S, S)
    group.set_kv_chunks([k[None] for k in ks], [v[None] for v in vs])
    b = proAttention(0, group).attn(q[None], ks[0][None], vs[0][None])
    torch.cuda.synchronize()
    assert tuple(a.shape) == (S, H, D) and torch.equal(a, b[0])
    # no sequence lengths at all: the dense path (core/attention.py:252-254)
    c = proAttention(0, group).varlen_attn(q[None], ks[0][None], vs[0][None])
    assert torch.equal(c, b)


def _cu(values, on_device):
    """cu_seqlens as the callers make them: int32, on the GPU (hunyuan_transformer.py:789-792) or on the host."""
    return torch.tensor(values, dtype=torch.int32, device="cuda" if on_device else "cpu")


class _no_host_sync:
    """Inside: any torch operation that blocks the host on the GPU raises (reading a device tensor's values,
    a pageable copy...).  The calling convention with device-resident boundaries promises there is none."""

    def __init__(self, on):
        self.on = on

    def __enter__(self):
        if self.on:
            torch.cuda.set_sync_debug_mode("error")

    def __exit__(self, *exc):
        torch.cuda.set_sync_debug_mode("default")
        return False


@pytest.mark.parametrize("cu_on_device", [False, True])
def test_varlen_stride_mode_matches_numeric_oracle(env, hip, cu_on_device):
    """Two segments per sample (valid tokens | padding), different boundaries in every chunk,
    over a divider sequence with reuse, coarsening and a full refresh.  With the boundaries on the GPU
    (the reference's calling convention) the call must not synchronise with the device."""
    from ditango_amd.core.attention import proAttention
    from ditango_amd.core.parallel_state import get_usp_group
    from ditango_amd.utils import update_timestep
    N, rank, H, D = 4, 2, 2, 128
    col = (1, 1, 1, 4, 4, 2, 2, 1, 1)
    T = len(col)
    rm = env(N, rank, T, 1)
    rm.divider_map[:, 0] = torch.tensor(col)
    curr, nxt = strides_from_dividers(N, col)
    total_q = 180
    cu_q = [0, 150, 180]
    lens = [170, 181, 160, 175]
    cu_k = [[0, 140, 170], [0, 150, 181], [0, 131, 160], [0, 150, 175]]
    g = torch.Generator().manual_seed(31)
    q = torch.randn(total_q, H, D, generator=g)
    ks = [torch.randn(n, H, D, generator=g) for n in lens]
    vs = [torch.randn(n, H, D, generator=g) for n in lens]
    state = {}

    def attn_fn(r, c):
        if r != rank:
            return (c,)
        o, l = om.varlen_chunk_attention(state["q"], state["ks"][c], state["vs"][c], cu_q, cu_k[c])
        return (o[None], l[None])

    def merge_fn(a, b):
        if isinstance(b[0], int):
            return tuple(b) if a is None else tuple(a) + tuple(b)
        return om.update_out_and_lse(None if a is None else a[0], None if a is None else a[1], b[0], b[1])

    def store_fn(s):
        return s if isinstance(s[0], int) else (om.bf16_round(s[0]), s[1])

    ring = RingOracle(N, attn_fn=attn_fn, merge_fn=merge_fn, store_fn=store_fn)
    group = get_usp_group()
    attn = proAttention(0, group)
    for t in range(T):
        print(f"case varlen t={t} curr={curr[t]} next={nxt[t]}", flush=True)
        qb, kb, vb = q.bfloat16(), [k.bfloat16() for k in ks], [v.bfloat16() for v in vs]
        state.update(q=qb, ks=kb, vs=vb)
        tr = ring.call(t, curr[t], nxt[t])[rank]
        update_timestep(t)
        dk, dv = [k.cuda() for k in kb], [v.cuda() for v in vb]
        dq, d_cu_q, d_cu_k = qb.cuda(), _cu(cu_q, cu_on_device), [_cu(c, cu_on_device) for c in cu_k]
        group.set_kv_chunks(dk, dv, cu_seqlens_kv=d_cu_k)
        torch.cuda.synchronize()
        with _no_host_sync(cu_on_device and t > 0):     # (the first call sets kernel attributes and allocates the workspace)
            out = attn.varlen_attn(dq, dk[rank], dv[rank], d_cu_q, d_cu_k[rank], max(150, 30), max(lens))
        torch.cuda.synchronize()
        assert attn.last_plan.computed == tr.computed and attn.last_plan.stores == tr.stores
        ref_out, ref_lse = tr.out
        err = (out.cpu() - ref_out[0]).abs().max().item()
        lerr = (attn.last_lse.cpu().squeeze(-1)[0].transpose(0, 1) - ref_lse.squeeze(-1)[0].transpose(0, 1)).abs().max().item()
        print(f"  out max-abs {err:.3e} lse {lerr:.3e}", flush=True)
        assert err <= OUT_TOL and lerr <= LSE_TOL
        q = q + 0.01 * torch.randn(q.shape, generator=g)
        ks = [k + 0.01 * torch.randn(k.shape, generator=g) for k in ks]
        vs = [v + 0.01 * torch.randn(v.shape, generator=g) for v in vs]


@pytest.mark.parametrize("cu_on_device", [False, True])
def test_varlen_mask_mode_matches_numeric_oracle(env, hip, cu_on_device):
    """The packed entry under a per-chunk reuse mask: every scheduled chunk runs once per segment
    (dt_attn_sched_seg_fwd, or dt_attn_sched_varlen_fwd when the boundaries are device tensors) into its
    cache slot; a trailing pad region belongs to no segment."""
    import numpy as np
    from oracle import mask_schedule as ms
    from ditango_amd.core.attention import proAttention
    from ditango_amd.core.parallel_state import get_usp_group
    from ditango_amd.utils import update_timestep
    C, diag, H, D, T = 5, 1, 2, 128, 5
    rm = env(C, diag, T, 1)
    mask = ms.seeded_mask(T, 1, C, 0.5, seed=3, diag=diag)
    rm.set_chunk_mask(mask, diag=diag)
    total_q = 300
    cu_q = [0, 260, 290]                # rows 290..299 belong to no segment
    lens = [270, 300, 64, 129, 200]
    cu_k = [[0, 200, 270], [0, 260, 300], [0, 64, 64], [0, 100, 129], [0, 0, 200]]   # empty segments included
    g = torch.Generator().manual_seed(41)
    q = torch.randn(total_q, H, D, generator=g)
    ks = [torch.randn(n, H, D, generator=g) for n in lens]
    vs = [torch.randn(n, H, D, generator=g) for n in lens]
    oracle = ms.MaskCacheOracle(C, diag)
    group = get_usp_group()
    attn = proAttention(0, group)
    for t in range(T):
        qb, kb, vb = q.bfloat16(), [k.bfloat16() for k in ks], [v.bfloat16() for v in vs]
        (ref_out, ref_lse), c_ids, r_ids = oracle.call(
            mask[t, 0], lambda c: om.varlen_chunk_attention(qb, kb[c], vb[c], cu_q, cu_k[c]),
            lambda sts: tuple(x[0] for x in om.merge_states_closed_form([s[0][None] for s in sts], [s[1][None] for s in sts])),
            lambda s: (om.bf16_round(s[0]), s[1]))
        print(f"case varlen mask t={t} computes {c_ids} reuses {r_ids}", flush=True)
        update_timestep(t)
        dk, dv = [k.cuda() for k in kb], [v.cuda() for v in vb]
        dq, d_cu_q, d_cu_k = qb.cuda(), _cu(cu_q, cu_on_device), [_cu(c, cu_on_device) for c in cu_k]
        group.set_kv_chunks(dk, dv, cu_seqlens_kv=d_cu_k)
        torch.cuda.synchronize()
        with _no_host_sync(cu_on_device and t > 0):
            out = attn.varlen_attn(dq, dk[diag], dv[diag], d_cu_q, d_cu_k[diag], 260, 300)
        torch.cuda.synchronize()
        n = int(rm.sched_counts_host[t, 0, 0])
        assert rm.sched_compute_ids[t, 0, :n].tolist() == list(c_ids)
        out = out.cpu()
        assert (out[cu_q[-1]:] == 0).all()
        err = (out[:cu_q[-1]] - ref_out[:cu_q[-1]]).abs().max().item()
        lse = attn.last_lse.cpu()[0, :cu_q[-1], :, 0].transpose(0, 1)
        lerr = (lse - ref_lse[:, :cu_q[-1]]).abs().max().item()
        print(f"  out max-abs {err:.3e} lse {lerr:.3e}", flush=True)
        assert err <= OUT_TOL and lerr <= LSE_TOL
        q = q + 0.01 * torch.randn(q.shape, generator=g)
        ks = [k + 0.01 * torch.randn(k.shape, generator=g) for k in ks]
        vs = [v + 0.01 * torch.randn(v.shape, generator=g) for v in vs]


def test_sched_seg_with_one_full_segment_is_the_dense_launch(hip):
    C, B, H, D, Sq = 3, 1, 2, 64, 130
    g = torch.Generator().manual_seed(5)
    q = torch.randn(B, Sq, H, D, generator=g).bfloat16().cuda()
    lens = [70, 128, 33]
    ks = [torch.randn(B, n, H, D, generator=g).bfloat16().cuda() for n in lens]
    vs = [torch.randn(B, n, H, D, generator=g).bfloat16().cuda() for n in lens]
    table = hip.ChunkTable(ks, vs)
    ids = torch.tensor([2, 0, 1], dtype=torch.int32, device="cuda")
    cnt = torch.tensor([3], dtype=torch.int32, device="cuda")

    def run(**kw):
        ao = torch.zeros(C, B, Sq, H, D, dtype=torch.bfloat16, device="cuda")
        al = torch.zeros(C, B, H, Sq, device="cuda")
        hip.attn_sched_fwd(q, table, ids, cnt, C, ao, al, -1, None, None, **kw)
        torch.cuda.synchronize()
        return ao, al

    a0, l0 = run()
    a1, l1 = run(seg_q=[(0, Sq)], seg_kv=[[(0, n)] for n in lens])
    assert torch.equal(a0, a1) and torch.equal(l0, l1)
    with pytest.raises(hip.DitangoHipError):
        run(seg_q=[(0, Sq + 1)], seg_kv=[[(0, n)] for n in lens])
    with pytest.raises(hip.DitangoHipError):
        run(seg_q=[(0, Sq)], seg_kv=[[(5, n)] for n in lens])
