"""IEEE-half tensors through every kernel of the path, against the CPU oracle on the same fp16 inputs.

``flash_attn_func`` takes fp16 as well as bf16 and the reference hands it whatever dtype the model runs in
(core/attention.py:137-143; executor/hunyuanvideo offers ``--precision fp16``).  fp16 tensors run on the fp16
MFMA with fp16 states and cache slots -- they are not rounded to bf16 on the way in.

Bar: lse max-abs <= 1e-3 as for bf16.  ``out`` is held to 4e-3 max-abs here, five times tighter than the bf16
bar: P and the output carry 11 significant bits instead of 8, and a path that rounded anything to bf16 in
between would not meet it (``test_fp16_is_not_rounded_through_bf16`` measures exactly that).
"""
import math

import numpy as np
import pytest
import torch

from oracle import attention_math as om
from oracle import mask_schedule as ms
from oracle import producer as P
from oracle.state_machine import RingOracle, strides_from_dividers

pytestmark = pytest.mark.gpu

OUT_TOL, LSE_TOL = 4e-3, 1e-3


def _half(t):
    return t.to(torch.float16)


def f16_round(x):
    return x.to(torch.float16).to(torch.float32)


def _check(out, lse, ref_out, ref_lse, what, out_tol=OUT_TOL):
    out, lse = out.float().cpu(), lse.float().cpu()
    err = (out - ref_out).abs().max().item()
    lerr = (lse - ref_lse).abs().max().item()
    rel = (out - ref_out).norm().item() / max(ref_out.norm().item(), 1e-30)
    print(f"{what}: out max-abs {err:.3e} rel-l2 {rel:.3e} lse max-abs {lerr:.3e}", flush=True)
    assert err <= out_tol and lerr <= LSE_TOL and rel <= 2e-3, what


@pytest.mark.parametrize("B,Sq,Sk,H,D,scale", [
    (1, 128, 64, 1, 128, 1.0),
    (1, 100, 77, 3, 128, 1.0),      # ragged Sq and Sk
    (2, 257, 333, 2, 128, 1.0),     # batch > 1, several tiles
    (1, 1, 1, 1, 128, 1.0),
    (2, 190, 201, 3, 64, 1.0),
    (1, 33, 1000, 2, 64, 1.0),
    (1, 300, 700, 2, 128, 6.0),     # scores of +-70 and more: tiles are redone with their exact maximum, P stays finite in fp16
    (1, 300, 700, 2, 64, 8.0),
])
def test_chunk_attention_fp16_matches_oracle(hip, B, Sq, Sk, H, D, scale):
    print(f"case fp16 chunk B={B} Sq={Sq} Sk={Sk} H={H} D={D} scale={scale}", flush=True)
    g = torch.Generator().manual_seed(B * 1000 + Sq + Sk + D)
    q = _half(torch.randn(B, Sq, H, D, generator=g) * scale)
    k = _half(torch.randn(B, Sk, H, D, generator=g))
    v = _half(torch.randn(B, Sk, H, D, generator=g))
    ref_out, ref_lse = om.chunk_attention(q, k, v)
    out, lse = hip.attn_chunk_fwd(q.cuda(), k.cuda(), v.cuda())
    torch.cuda.synchronize()
    assert out.dtype == torch.float16 and torch.isfinite(out.float()).all()
    _check(out, lse, ref_out, ref_lse, "fp16 chunk")


def test_fp16_is_not_rounded_through_bf16(hip):
    """The distance to fp32 attention of the fp16 inputs is that of an fp16 pipeline (P and out rounded to 11
    bits), an order of magnitude under what rounding q / k / v to bf16 first costs on the same data."""
    B, Sq, Sk, H, D = 1, 256, 512, 2, 128
    g = torch.Generator().manual_seed(5)
    q, k, v = (_half(torch.randn(B, n, H, D, generator=g)) for n in (Sq, Sk, Sk))
    ref_out, ref_lse = om.chunk_attention(q, k, v)
    out, lse = hip.attn_chunk_fwd(q.cuda(), k.cuda(), v.cuda())
    o16 = hip.attn_chunk_fwd(q.cuda().bfloat16(), k.cuda().bfloat16(), v.cuda().bfloat16())
    torch.cuda.synchronize()
    e_native = (out.float().cpu() - ref_out).abs().max().item()
    e_lse = (lse.cpu() - ref_lse).abs().max().item()
    e_rounded = (o16[0].float().cpu() - ref_out).abs().max().item()
    l_rounded = (o16[1].cpu() - ref_lse).abs().max().item()
    print(f"native fp16: out {e_native:.2e} lse {e_lse:.2e}; through bf16: out {e_rounded:.2e} lse {l_rounded:.2e}", flush=True)
    assert e_native <= 1e-3 and e_lse <= 2e-4
    assert e_rounded > 3 * e_native and l_rounded > 3 * e_lse


def test_fp16_and_bf16_do_not_mix_and_prescaled_is_bf16_only(hip):
    B, S, H, D = 1, 64, 1, 128
    q = torch.zeros(B, S, H, D, dtype=torch.float16, device="cuda")
    kb = torch.zeros(B, S, H, D, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(hip.DitangoHipError):
        hip.attn_chunk_fwd(q, kb, kb)
    table = hip.ChunkTable([q], [q])
    o, l = torch.empty_like(q), torch.empty(B, H, S, device="cuda")
    with pytest.raises(hip.DitangoHipError):
        hip.attn_jobs_fwd(q, table, [[0]], [o], [l], q_prescaled=True)
    with pytest.raises(hip.DitangoHipError):
        hip.attn_jobs_fwd(q, table, [[0]], [o.bfloat16()], [l])           # states are written in q's dtype
    # the C entry point refuses the flag combination itself
    lib = hip.load_library()
    import ctypes
    kp, vp = (ctypes.c_void_p * 1)(q.data_ptr()), (ctypes.c_void_p * 1)(q.data_ptr())
    lens, sbs = (ctypes.c_int32 * 1)(S), (ctypes.c_int64 * 1)(q.stride(0))
    begin, chunks = (ctypes.c_int32 * 2)(0, 1), (ctypes.c_int32 * 1)(0)
    outs, lses = (ctypes.c_void_p * 1)(o.data_ptr()), (ctypes.c_void_p * 1)(l.data_ptr())
    rc = lib.dt_attn_seg_jobs_ws_fwd(q.data_ptr(), B, S, H, D, q.stride(0), q.stride(1), q.stride(2), 1, kp, vp, lens, sbs,
                                     q.stride(1), q.stride(2), 1, begin, chunks, None, None, None, None, outs, lses, 0.0,
                                     hip.DT_ATTN_Q_PRESCALED | hip.DT_ATTN_FP16, None, 0, None)
    assert rc == -2 and b"fp16" in lib.dt_last_error()
    torch.cuda.synchronize()


@pytest.mark.parametrize("D,lens", [(128, [2000, 1500]), (64, [1100, 900, 40])])
def test_jobs_with_tail_split_and_fold_in_fp16(hip, D, lens):
    """Several states per launch with the tail of the launch split over the workspace (partial states in fp16, fold
    kernel) against the oracle, and against the same launch without a workspace."""
    B, H, Sq = 1, 24, 3000
    dev = "cuda"
    g = torch.Generator().manual_seed(D)
    q = _half(torch.randn(B, Sq, H, D, generator=g))
    ks = [_half(torch.randn(B, n, H, D, generator=g)) for n in lens]
    vs = [_half(torch.randn(B, n, H, D, generator=g)) for n in lens]
    table = hip.ChunkTable([k.to(dev) for k in ks], [v.to(dev) for v in vs])
    jobs = [[c] for c in range(len(lens))]

    def run(**how):
        o = [torch.zeros(B, Sq, H, D, dtype=torch.float16, device=dev) for _ in jobs]
        l = [torch.zeros(B, H, Sq, device=dev) for _ in jobs]
        hip.attn_jobs_fwd(q.to(dev), table, jobs, o, l, **how)
        torch.cuda.synchronize()
        return o, l

    plain = run()
    split = run(workspace=hip.attn_workspace(dev))
    scratch = run(no_alloc=True)
    heads = [0, 11, 23]
    for c in range(len(lens)):
        ref_out, ref_lse = om.chunk_attention(q[:, :, heads], ks[c][:, :, heads], vs[c][:, :, heads])
        for name, (o, l) in (("plain", plain), ("workspace", split), ("library scratch", scratch)):
            _check(o[c][:, :, heads], l[c][:, heads], ref_out, ref_lse, f"D={D} chunk {c} {name}")
    if D == 128:
        assert any(not torch.equal(a, b) for a, b in zip(split[0], plain[0])), "the tail was expected to be split"


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("n,kinds", [(3, "hhh"), (6, "hhhhhh"), (9, "hhhhhhhhh"), (5, "hbfhb"), (2, "fh")])
@pytest.mark.parametrize("dst", [torch.float32, torch.float16])
def test_merge_of_fp16_states_matches_closed_form(hip, D, n, kinds, dst):
    """All-fp16 launches (their own decode path), and fp16 mixed with bf16 and fp32 states; fp32 and fp16 results."""
    B, S, H = 2, 77, 4
    g = torch.Generator().manual_seed(n * 7 + D)
    dt = {"h": torch.float16, "b": torch.bfloat16, "f": torch.float32}
    outs = [torch.randn(B, S, H, D, generator=g).to(dt[c]) for c in kinds]
    lses = [torch.randn(B, H, S, generator=g) * 3 for _ in kinds]
    lses[0][0, 0, :5] = -math.inf
    ref_out, ref_lse = om.merge_states_closed_form([o.float() for o in outs], lses)
    out, lse = hip.merge_states([o.cuda() for o in outs], [l.cuda() for l in lses], dst_dtype=dst)
    torch.cuda.synchronize()
    assert out.dtype == dst
    tol = 1e-5 * n if dst == torch.float32 else 2.0 ** -11 * float(ref_out.abs().max()) * 1.01 + 1e-5 * n
    assert (out.float().cpu() - ref_out).abs().max().item() <= tol
    finite = torch.isfinite(ref_lse)
    assert (lse.cpu()[finite] - ref_lse[finite]).abs().max().item() <= 1e-5


@pytest.mark.parametrize("D,H", [(128, 3), (64, 8), (64, 3)])
def test_cache_store_and_load_with_fp16_slots(hip, D, H):
    B, S = 1, 150
    g = torch.Generator().manual_seed(D + H)
    src = torch.randn(B, S, H, D, generator=g)
    lse = torch.randn(B, H, S, generator=g)
    slot_o = torch.empty(B, S, H, D, dtype=torch.float16, device="cuda")
    slot_l = torch.empty(B, H, S, device="cuda")
    # fp32 state (running layout of the lse) -> fp16 slot: one rounding to nearest even
    hip.cache_store(src.cuda(), lse.transpose(1, 2).contiguous().unsqueeze(-1).cuda(), slot_o, slot_l)
    torch.cuda.synchronize()
    assert torch.equal(slot_o.cpu(), src.half()) and torch.equal(slot_l.cpu(), lse)
    # fp16 state -> fp16 slot: a flat copy
    slot2_o, slot2_l = torch.empty_like(slot_o), torch.empty_like(slot_l)
    hip.cache_store(slot_o, slot_l, slot2_o, slot2_l)
    # fp16 slot -> fp32 / bf16 / fp16 tensors
    wide, wl = hip.cache_load(slot2_o, slot2_l, torch.float32, dst_lse_bsh=True)
    narrow, _ = hip.cache_load(slot2_o, slot2_l, torch.bfloat16)
    same, _ = hip.cache_load(slot2_o, slot2_l, torch.float16)
    torch.cuda.synchronize()
    assert torch.equal(wide.cpu(), src.half().float()) and torch.equal(wl.cpu().squeeze(-1).transpose(1, 2), lse)
    assert torch.equal(narrow.cpu(), src.half().float().bfloat16()) and torch.equal(same.cpu(), src.half())


@pytest.mark.parametrize("D,norm,rope", [(128, P.NORM_RMS, P.ROPE_INTERLEAVED), (64, P.NORM_LAYER, P.ROPE_INTERLEAVED),
                                         (128, P.NORM_RMS, P.ROPE_HALVES), (64, P.NORM_NONE, P.ROPE_NONE)])
@pytest.mark.parametrize("rounding", [0, P.ROUND_NORM_BF16 | P.ROUND_ROPE_BF16])
def test_producer_on_fp16_activations(hip, D, norm, rope, rounding):
    """QK-norm + RoPE reading and writing fp16; with the eager-rounding bits the intermediate roundings are to fp16."""
    B, S, H = 2, 37, 5
    g = torch.Generator().manual_seed(D + norm + rope)
    x = (torch.randn(B, S, H, D, generator=g) * 2.0 + 0.3).half()
    w, b = torch.rand(D, generator=g) + 0.5, torch.randn(D, generator=g) * 0.1
    cos = sin = None
    secs = ()
    if rope != P.ROPE_NONE:
        th = torch.rand(S, D // 2, generator=g) * 2 * math.pi
        if rope == P.ROPE_INTERLEAVED:
            cos, sin = th.cos().repeat_interleave(2, -1).contiguous(), th.sin().repeat_interleave(2, -1).contiguous()
        else:
            cos, sin = torch.cat((th.cos(), th.cos()), -1).contiguous(), torch.cat((th.sin(), th.sin()), -1).contiguous()
    o = P.qk_norm_rope(x, norm, w, b, 1e-6, rope, cos, sin, 0, S, secs, rounding)
    y = hip.qk_norm_rope(x.cuda(), norm=norm, weight=w.cuda(), bias=b.cuda(), eps=1e-6, rope=rope,
                         cos=None if cos is None else cos.cuda(), sin=None if sin is None else sin.cuda(), rounding=rounding)
    torch.cuda.synchronize()
    assert y.dtype == torch.float16 and y.is_contiguous()
    err = (y.float().cpu() - o).abs()
    if rounding == 0:
        # fp32 math, one rounding: within half an fp16 ulp of the oracle's fp32 value (+ summation-order slack)
        assert not bool((err > o.abs() * 2.0 ** -11 * 1.001 + 3e-5).any())
    else:
        same = (y.cpu() == o.half()).float().mean().item()
        assert same > 0.99 and float(err.max()) <= 2.0 ** -9 * float(o.abs().max())


@pytest.fixture
def env(hip):
    from ditango_amd.core import config, parallel_state, redundancy_map as rmod
    from ditango_amd import utils

    def make(N, rank, T, L, **cfg):
        parallel_state.init_local_groups(N, rank)
        config.init_config(None, num_inference_steps=T, num_layers=L, **cfg)
        rmod.destroy_redundancy_map()
        rmod._redundancy_map = rmod.RedundancyMap(config.get_config())
        return rmod.get_redundancy_map()

    yield make
    rmod.destroy_redundancy_map()
    parallel_state.destroy_local_groups()
    utils.update_timestep(0)


def _perturb(x, g):
    return x + 0.01 * torch.randn(x.shape, generator=g)


def _cmp(out, lse_bsh1, ref_out, ref_lse_bhs, what):
    _check(out, lse_bsh1.cpu().squeeze(-1).transpose(1, 2), ref_out, ref_lse_bhs, what)


@pytest.mark.parametrize("N,rank,D,col", [
    (4, 1, 128, (1, 1, 1, 2, 2, 2, 1, 4, 2, 2, 1, 1)),
    (8, 3, 64, (1, 1, 1, 4, 4, 4, 2, 2, 2, 2, 1, 1)),
])
def test_stride_mode_in_fp16_matches_numeric_oracle(env, N, rank, D, col):
    """The reference's own mode on fp16 tensors: schedule, stores and pointer exact, numerics against the lock-step
    oracle whose cached states are rounded to fp16 (what the fp16 slots hold)."""
    from ditango_amd.core.attention import proAttention
    from ditango_amd.core.parallel_state import get_usp_group
    from ditango_amd.utils import update_timestep

    T, B, H, S = len(col), 1, 2, 100
    rm = env(N, rank, T, 1)
    rm.divider_map[:, 0] = torch.tensor(col)
    curr, nxt = strides_from_dividers(N, col)
    g = torch.Generator().manual_seed(17)
    q = torch.randn(B, S, H, D, generator=g)
    ks = [torch.randn(B, S, H, D, generator=g) for _ in range(N)]
    vs = [torch.randn(B, S, H, D, generator=g) for _ in range(N)]
    state = {}

    def attn_fn(r, c):
        if r != rank:
            return (c,)
        return om.chunk_attention(state["q"], state["ks"][c], state["vs"][c])

    def merge_fn(a, b):
        if isinstance(b[0], int):
            return tuple(b) if a is None else tuple(a) + tuple(b)
        return om.update_out_and_lse(None if a is None else a[0], None if a is None else a[1], b[0], b[1])

    def store_fn(s):
        return s if isinstance(s[0], int) else (f16_round(s[0]), s[1])

    ring = RingOracle(N, attn_fn=attn_fn, merge_fn=merge_fn, store_fn=store_fn)
    group = get_usp_group()
    attn = proAttention(0, group)
    for t in range(T):
        print(f"case fp16 stride N={N} rank={rank} D={D} t={t} curr={curr[t]} next={nxt[t]}", flush=True)
        qh, kh, vh = _half(q), [_half(k) for k in ks], [_half(v) for v in vs]
        state.update(q=qh, ks=kh, vs=vh)
        tr = ring.call(t, curr[t], nxt[t])[rank]
        update_timestep(t)
        dk, dv = [k.cuda() for k in kh], [v.cuda() for v in vh]
        group.set_kv_chunks(dk, dv)
        out = attn.attn(qh.cuda(), dk[rank], dv[rank])
        torch.cuda.synchronize()
        p = attn.last_plan
        assert p.computed == tr.computed and p.reuse_merged == tr.reuse_merged and p.stores == tr.stores
        assert p.target_after == tr.target_after and p.occupancy_after == tr.occupancy_after
        assert out.dtype == torch.float32
        assert all(o is None or o.dtype == torch.float16 for o in attn.cache.out_block_cache)
        ref_out, ref_lse = tr.out
        _cmp(out, attn.last_lse, ref_out, ref_lse.squeeze(-1).transpose(1, 2), f"t={t}")
        q, ks, vs = _perturb(q, g), [_perturb(k, g) for k in ks], [_perturb(v, g) for v in vs]


@pytest.mark.parametrize("C,diag,D,lens", [(8, 5, 64, None), (6, -1, 128, [70, 69, 69, 70, 1, 64])])
def test_mask_mode_in_fp16_matches_numeric_oracle(env, C, diag, D, lens):
    """The device-scheduled launch writing fp16 states into an fp16 arena, merged with the cached ones."""
    from ditango_amd.core.attention import proAttention
    from ditango_amd.core.parallel_state import get_usp_group
    from ditango_amd.utils import update_timestep

    T, L, B, H, Sq = 4, 2, 1, 3, 90
    lens = lens or [Sq] * C
    rank = max(diag, 0)
    rm = env(C, rank, T, L)
    mask = ms.seeded_mask(T, L, C, 0.6, seed=C + D, diag=diag)
    rm.set_chunk_mask(mask, diag=diag)
    group = get_usp_group()
    layers = [proAttention(l, group) for l in range(L)]
    oracles = [ms.MaskCacheOracle(C, diag) for _ in range(L)]
    g = torch.Generator().manual_seed(23)
    q = torch.randn(B, Sq, H, D, generator=g)
    ks = [torch.randn(B, n, H, D, generator=g) for n in lens]
    vs = [torch.randn(B, n, H, D, generator=g) for n in lens]
    for t in range(T):
        update_timestep(t)
        for l in range(L):
            print(f"case fp16 mask C={C} diag={diag} D={D} t={t} l={l}", flush=True)
            qh, kh, vh = _half(q), [_half(k) for k in ks], [_half(v) for v in vs]
            (ref_out, ref_lse), _, _ = oracles[l].call(
                mask[t, l], lambda c: om.chunk_attention(qh, kh[c], vh[c]),
                lambda sts: om.merge_states_closed_form([s[0] for s in sts], [s[1] for s in sts]),
                lambda s: (f16_round(s[0]), s[1]))
            dk, dv = [k.cuda() for k in kh], [v.cuda() for v in vh]
            group.set_kv_chunks(dk, dv)
            layers[l].out_dtype = torch.float16 if l == 1 else torch.float32     # the merge can write the model's dtype
            out = layers[l].attn(qh.cuda(), dk[rank], dv[rank])
            torch.cuda.synchronize()
            assert layers[l].cache.arena_out.dtype == torch.float16 and out.dtype == layers[l].out_dtype
            _cmp(out, layers[l].last_lse, ref_out, ref_lse, f"t={t} l={l}")
            q, ks, vs = _perturb(q, g), [_perturb(k, g) for k in ks], [_perturb(v, g) for v in vs]


def test_varlen_with_device_boundaries_in_fp16(env):
    """HunyuanVideo's entry on fp16 tensors: packed batch, int32 cu_seqlens on the GPU, no host read of them."""
    from ditango_amd.core.attention import proAttention
    from ditango_amd.core.parallel_state import get_usp_group
    N, rank, H, D, total = 2, 0, 3, 128, 400
    env(N, rank, 1, 1)
    g = torch.Generator().manual_seed(31)
    q = _half(torch.randn(total, H, D, generator=g))
    ks = [_half(torch.randn(total, H, D, generator=g)) for _ in range(N)]
    vs = [_half(torch.randn(total, H, D, generator=g)) for _ in range(N)]
    cu_q = [0, 330, 400]
    cu_k = [[0, 280, 400], [0, 310, 390]]
    group = get_usp_group()
    dk, dv = [k.cuda() for k in ks], [v.cuda() for v in vs]
    dcu = [torch.tensor(c, dtype=torch.int32, device="cuda") for c in cu_k]
    group.set_kv_chunks(dk, dv, cu_seqlens_kv=dcu)
    attn = proAttention(0, group)
    dq, dcq = q.cuda(), torch.tensor(cu_q, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    torch.cuda.set_sync_debug_mode("error")
    try:
        out = attn.varlen_attn(dq, dk[rank], dv[rank], dcq, dcu[rank], 330, 310)
    finally:
        torch.cuda.set_sync_debug_mode("default")
    torch.cuda.synchronize()
    states = [om.varlen_chunk_attention(q, ks[c], vs[c], cu_q, cu_k[c]) for c in range(N)]
    ref_out, ref_lse = om.merge_states_closed_form([s[0][None] for s in states], [s[1][None] for s in states])
    lse = attn.last_lse.cpu().squeeze(-1).transpose(1, 2)
    _check(out[None], lse, ref_out, ref_lse, "fp16 varlen")
