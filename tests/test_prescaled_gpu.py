"""The opt-in mode in which the caller has folded ``softmax_scale * log2(e)`` into q
(``DT_ATTN_Q_PRESCALED``): the kernels then take ``q k^T`` as exponents of 2 and keep the
reference 0 for rows of moderate scores.

The oracle needs no such mode: with the prescaled q and ``scale = ln 2`` the textbook closed form
IS what the kernel must return (``exp(s ln 2) = 2^s``).  Same bar as everywhere: out max-abs
<= 2e-2, lse <= 1e-3 (relative to max(1, |lse|) where the scores are made huge on purpose).
"""
import ctypes
import math

import numpy as np
import pytest
import torch

from oracle import attention_math as om
from oracle import producer as P

pytestmark = pytest.mark.gpu

LN2 = math.log(2.0)


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


def _check(out, lse, ref_out, ref_lse, what):
    out, lse = out.float().cpu(), lse.float().cpu()
    err = (out - ref_out).abs().max().item()
    fin = torch.isfinite(ref_lse)
    assert bool((torch.isfinite(lse) == fin).all()), f"{what}: -inf pattern of the lse differs"
    lerr = ((lse[fin] - ref_lse[fin]).abs() / ref_lse[fin].abs().clamp(min=1.0)).max().item() if bool(fin.any()) else 0.0
    print(f"{what}: out max-abs {err:.3e} lse {lerr:.3e}", flush=True)
    assert err <= 2e-2 and lerr <= 1e-3, f"{what}: out {err} lse {lerr}"


def _fold(q, D):
    """What a caller does: one rounding to bf16 AFTER the multiplication."""
    return (q * (D ** -0.5 * math.log2(math.e))).bfloat16()


@pytest.mark.parametrize("B,Sq,Sk,H,D", [
    (1, 128, 64, 1, 128), (2, 257, 333, 2, 128), (1, 1, 1, 1, 128), (1, 100, 77, 3, 64), (1, 33, 1000, 2, 64),
    (1, 300, 2610, 2, 128),
])
def test_chunk_attention_with_prescaled_q(hip, B, Sq, Sk, H, D):
    print(f"case prescaled B={B} Sq={Sq} Sk={Sk} H={H} D={D}", flush=True)
    g = torch.Generator().manual_seed(Sq * 7 + Sk + D)
    q = _fold(torch.randn(B, Sq, H, D, generator=g), D)
    k = torch.randn(B, Sk, H, D, generator=g).bfloat16()
    v = torch.randn(B, Sk, H, D, generator=g).bfloat16()
    ref = om.chunk_attention(q, k, v, scale=LN2)
    out = torch.empty(B, Sq, H, D, dtype=torch.bfloat16, device="cuda")
    lse = torch.empty(B, H, Sq, device="cuda")
    hip.attn_jobs_fwd(q.cuda(), hip.ChunkTable([k.cuda()], [v.cuda()]), [[0]], [out], [lse], q_prescaled=True)
    torch.cuda.synchronize()
    _check(out, lse, *ref, "prescaled chunk")


@pytest.mark.parametrize("D", [64, 128])
def test_rows_that_leave_the_band_of_the_zero_reference(hip, D):
    """Rows whose scores are huge (the reference must rise), hugely negative (2^s would underflow with
    reference 0), growing from tile to tile (the sum runs over 2^40 later on), and rows of an ordinary
    wavefront next to them; several chunks in one job, a ragged last tile, an empty chunk."""
    print(f"case prescaled band D={D}", flush=True)
    B, Sq, H = 1, 700, 2
    lens = [1000, 0, 333]
    g = torch.Generator().manual_seed(D)
    q = torch.randn(B, Sq, H, D, generator=g) * (D ** -0.5 * math.log2(math.e))
    q[:, 100:200] *= 12.0
    q[:, 300:330] *= 40.0
    ks = [torch.randn(B, n, H, D, generator=g) for n in lens]
    ks[0][:, 500:] *= 3.0                                   # later tiles larger than the first
    ks[2] *= 6.0                                            # and the last chunk larger still
    vs = [torch.randn(B, n, H, D, generator=g).bfloat16() for n in lens]
    q[:, 400:420] = -2.0 / math.sqrt(D / 64)
    q[:, 420:440] = 2.0 / math.sqrt(D / 64)
    for k in ks:                                            # give those rows keys of one sign
        k[:, :, :, :] = torch.where(torch.rand(k.shape, generator=g) < 0.5, k, k.abs())
    q, ks = q.bfloat16(), [k.bfloat16() for k in ks]
    ref = om.full_attention(q.float() * LN2 * math.sqrt(D), [k for k in ks if k.shape[1]], [v for v in vs if v.shape[1]])
    out = torch.empty(B, Sq, H, D, dtype=torch.bfloat16, device="cuda")
    lse = torch.empty(B, H, Sq, device="cuda")
    table = hip.ChunkTable([k.cuda() for k in ks], [v.cuda() for v in vs])
    hip.attn_jobs_fwd(q.cuda(), table, [[0, 1, 2]], [out], [lse], q_prescaled=True)
    torch.cuda.synchronize()
    s_max = (torch.einsum("bqhd,bkhd->bhqk", q.float(), torch.cat(ks, 1).float())).abs().max().item()
    print(f"  largest |score| {s_max:.0f} (exponent of 2)", flush=True)
    assert s_max > 150
    _check(out, lse, *ref, "band")


def test_prescaled_and_scaled_inside_agree(hip):
    """The two modes differ only by where q is rounded."""
    B, Sq, Sk, H, D = 1, 200, 900, 3, 128
    g = torch.Generator().manual_seed(3)
    qf = torch.randn(B, Sq, H, D, generator=g)
    k = torch.randn(B, Sk, H, D, generator=g).bfloat16().cuda()
    v = torch.randn(B, Sk, H, D, generator=g).bfloat16().cuda()
    table = hip.ChunkTable([k], [v])
    o = [torch.empty(B, Sq, H, D, dtype=torch.bfloat16, device="cuda") for _ in range(2)]
    l = [torch.empty(B, H, Sq, device="cuda") for _ in range(2)]
    hip.attn_jobs_fwd(qf.bfloat16().cuda(), table, [[0]], [o[0]], [l[0]])
    hip.attn_jobs_fwd(_fold(qf, D).cuda(), table, [[0]], [o[1]], [l[1]], q_prescaled=True)
    torch.cuda.synchronize()
    assert (o[0].float() - o[1].float()).abs().max().item() <= 2e-2
    assert (l[0] - l[1]).abs().max().item() <= 2e-2          # two roundings of q: 2^-9 relative on the scores


def test_producer_folds_the_scale_and_the_layer_runs_prescaled(hip, env):
    """prepare_qk(fold_softmax_scale=...) -> proAttention.q_prescaled in mask mode (device-scheduled
    launch, cached states, merge), against the oracle on the oracle's own folded q."""
    from ditango_amd.core.attention import proAttention
    from ditango_amd.core.parallel_state import get_usp_group
    from ditango_amd.producer import folded_scale, prepare_qk
    from ditango_amd.utils import update_timestep

    C, B, H, D, Sq = 4, 1, 5, 64, 96
    rm = env(C, 0, 2, 1)
    mask = np.zeros((2, 1, C), dtype=np.uint8)
    mask[1, 0, 2] = 1                                         # second step reuses chunk 2
    rm.set_chunk_mask(mask, diag=0)
    g = torch.Generator().manual_seed(77)
    qkv = torch.randn(B, C * Sq, 3, H, D, generator=g).bfloat16()
    wq, wk = torch.rand(D, generator=g) + 0.5, torch.rand(D, generator=g) + 0.5
    c = folded_scale(D)
    assert abs(c - D ** -0.5 * math.log2(math.e)) < 1e-12
    qn = P.qk_norm_rope(qkv[:, :, 0], P.NORM_RMS, wq, None, 1e-6, out_scale=c).bfloat16()
    kn = P.qk_norm_rope(qkv[:, :, 1], P.NORM_RMS, wk, None, 1e-6).bfloat16()
    ref_out, ref_lse = om.chunk_attention(qn[:, :Sq], kn, qkv[:, :, 2], scale=LN2)
    dev = qkv.cuda()
    qd = prepare_qk(dev[:, :, 0], norm="rms", weight=wq, fold_softmax_scale=0.0)
    kd = prepare_qk(dev[:, :, 1], norm="rms", weight=wk)
    vd = prepare_qk(dev[:, :, 2])
    assert (qd.float().cpu() - qn.float()).abs().max().item() <= 2.0 ** -7 * qn.float().abs().max().item()
    group = get_usp_group()
    group.set_kv_chunks(list(kd.split(Sq, dim=1)), list(vd.split(Sq, dim=1)))
    layer = proAttention(0, group)
    layer.q_prescaled = True
    for t in range(2):
        update_timestep(t)
        out = layer.attn(qd[:, :Sq], kd[:, :Sq], vd[:, :Sq])
        torch.cuda.synchronize()
        lse = layer.last_lse.squeeze(-1).transpose(1, 2)
        _check(out, lse, ref_out, ref_lse, f"layer call, step {t}")


def test_unknown_flags_and_bad_out_scale_are_rejected(hip):
    lib = hip.load_library()
    B, Sq, H, D = 1, 8, 1, 128
    q = torch.zeros(B, Sq, H, D, dtype=torch.bfloat16, device="cuda")
    out = torch.full((B, Sq, H, D), 7.0, dtype=torch.bfloat16, device="cuda")
    lse = torch.zeros(B, H, Sq, device="cuda")
    table = hip.ChunkTable([q], [q])
    begin, chunks = (ctypes.c_int32 * 2)(0, 1), (ctypes.c_int32 * 1)(0)
    outs, lses = (ctypes.c_void_p * 1)(out.data_ptr()), (ctypes.c_void_p * 1)(lse.data_ptr())

    def call(flags):
        return lib.dt_attn_seg_jobs_ws_fwd(q.data_ptr(), B, Sq, H, D, q.stride(0), q.stride(1), q.stride(2), table.n,
                                           table.k_ptrs, table.v_ptrs, table.lens, table.sb, table.ss, table.sh,
                                           1, begin, chunks, None, None, None, None, outs, lses, ctypes.c_float(0.0),
                                           flags, None, 0, None)

    assert call(4) == -1 and b"flags" in lib.dt_last_error()       # 1 and 2 are DT_ATTN_Q_PRESCALED and DT_ATTN_FP16
    torch.cuda.synchronize()
    assert (out.float() == 7.0).all()
    assert call(hip.DT_ATTN_Q_PRESCALED) == 0
    x = torch.zeros(1, 4, 2, 128, dtype=torch.bfloat16, device="cuda")
    for bad in (0.0, -1.0, float("inf"), float("nan")):
        with pytest.raises(hip.DitangoHipError):
            hip.qk_norm_rope(x, out_scale=bad)


@pytest.mark.parametrize("D", [64, 128])
def test_producer_out_scale_matches_oracle(hip, D):
    B, S, H = 2, 37, 5
    g = torch.Generator().manual_seed(D)
    x = (torch.randn(B, S, H, D, generator=g) * 2.0 + 0.3).to(torch.bfloat16)
    w = torch.rand(D, generator=g) + 0.5
    th = torch.rand(S, D // 2, generator=g) * 6.28
    cos, sin = th.cos().repeat_interleave(2, -1).contiguous(), th.sin().repeat_interleave(2, -1).contiguous()
    c = D ** -0.5 * math.log2(math.e)
    o = P.qk_norm_rope(x, P.NORM_RMS, w, None, 1e-6, P.ROPE_INTERLEAVED, cos, sin, 0, S, (), 0, out_scale=c)
    y = hip.qk_norm_rope(x.cuda(), norm=P.NORM_RMS, weight=w.cuda(), rope=P.ROPE_INTERLEAVED, cos=cos.cuda(),
                         sin=sin.cuda(), out_scale=c)
    torch.cuda.synchronize()
    err = (y.float().cpu() - o).abs()
    assert bool((err <= o.abs() * 2.0 ** -8 * 1.001 + 3e-5).all())
