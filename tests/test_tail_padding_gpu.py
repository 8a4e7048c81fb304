"""Rows behind the end of a KV chunk (or of a segment's key range) must never reach the result.

The attention kernel brings K/V tiles in with raw buffer loads and relies on the hardware bounds
check to zero the rows of a last, partial tile.  Ordinary tests cannot see a hole in that: data
behind a chunk is finite, a masked key has probability 0, and 0 * finite = 0.  Here K and V are
views into larger buffers whose every other row holds NaN (behind the chunk, between and behind
the segments of a packed batch), with tail lengths on either side of the 32-row boundary between
the two halves of a tile.  The result must be finite and equal the oracle's.
"""
import pytest
import torch

from oracle import attention_math as om

pytestmark = pytest.mark.gpu
OUT_TOL, LSE_TOL = 2e-2, 1e-3


def _padded(B, S, H, D, g, pad):
    """A [B,S,H,D] bf16 view (rows [pad, pad+S)) of a NaN-filled [B, S + 2*pad, H, D] buffer; and its CPU copy."""
    x = torch.randn(B, S, H, D, generator=g).bfloat16()
    buf = torch.full((B, S + 2 * pad, H, D), float("nan"), dtype=torch.bfloat16, device="cuda")
    buf[:, pad:pad + S] = x.cuda()
    return x, buf[:, pad:pad + S]


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("Sk", [1, 17, 32, 33, 47, 63, 64 + 5, 64 + 40, 128 + 31, 128 + 32, 128 + 60, 64 * 9 + 5, 64 * 20 + 33])
def test_rows_behind_a_chunk_are_never_read_as_data(hip, D, Sk):
    B, Sq, H = 2, 70, 3
    print(f"case padding D={D} Sk={Sk}", flush=True)
    g = torch.Generator().manual_seed(1000 * D + Sk)
    q = torch.randn(B, Sq, H, D, generator=g).bfloat16()
    k, dk = _padded(B, Sk, H, D, g, 96)
    v, dv = _padded(B, Sk, H, D, g, 96)
    ref_out, ref_lse = om.chunk_attention(q, k, v)
    out, lse = hip.attn_chunk_fwd(q.cuda(), dk, dv)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all(), "NaN rows behind the chunk leaked"
    assert (out.float().cpu() - ref_out).abs().max().item() <= OUT_TOL
    assert (lse.cpu() - ref_lse).abs().max().item() <= LSE_TOL


@pytest.mark.parametrize("D", [64, 128])
def test_rows_between_segments_are_never_read_as_data(hip, D):
    """Jobs on key sub-ranges of one packed chunk: everything outside the ranges is NaN."""
    B, H = 1, 2
    g = torch.Generator().manual_seed(77 + D)
    total_k = 700
    ranges = [(5, 1), (40, 31), (100, 33), (200, 64 + 47), (400, 128 + 32), (600, 95)]   # (begin, length)
    k = torch.randn(B, total_k, H, D, generator=g).bfloat16()
    v = torch.randn(B, total_k, H, D, generator=g).bfloat16()
    live = torch.zeros(total_k, dtype=torch.bool)
    for b, n in ranges:
        live[b:b + n] = True
    dk, dv = k.cuda(), v.cuda()
    dk[:, ~live.cuda()] = float("nan")
    dv[:, ~live.cuda()] = float("nan")
    Sq = 50 * len(ranges)
    q = torch.randn(B, Sq, H, D, generator=g).bfloat16()
    table = hip.ChunkTable([dk], [dv])
    out = torch.zeros(B, Sq, H, D, dtype=torch.bfloat16, device="cuda")
    lse = torch.zeros(B, H, Sq, dtype=torch.float32, device="cuda")
    jobs = [[0]] * len(ranges)
    q_ranges = [(50 * i, 50) for i in range(len(ranges))]
    kv_ranges = [[r] for r in ranges]
    hip.attn_jobs_fwd(q.cuda(), table, jobs, [out] * len(ranges), [lse] * len(ranges), q_ranges=q_ranges,
                      kv_ranges=kv_ranges)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all(), "NaN rows outside a key range leaked"
    for i, (b, n) in enumerate(ranges):
        ro, rl = om.chunk_attention(q[:, 50 * i:50 * i + 50], k[:, b:b + n], v[:, b:b + n])
        assert (out[:, 50 * i:50 * i + 50].float().cpu() - ro).abs().max().item() <= OUT_TOL, f"segment {i}"
        assert (lse[:, :, 50 * i:50 * i + 50].cpu() - rl).abs().max().item() <= LSE_TOL, f"segment {i}"


@pytest.mark.parametrize("D", [64, 128])
def test_rows_behind_every_chunk_of_a_multi_chunk_job(hip, D):
    """One job over three chunks of ragged lengths (the tile cursor moves from chunk to chunk while V still loads
    from the previous one): NaN behind each of them."""
    B, Sq, H = 1, 300, 2
    g = torch.Generator().manual_seed(5 + D)
    q = torch.randn(B, Sq, H, D, generator=g).bfloat16()
    lens = [64 * 3 + 7, 40, 64 * 5 + 33]
    cpu, dev = [], []
    for n in lens:
        (k, dk), (v, dv) = _padded(B, n, H, D, g, 80), _padded(B, n, H, D, g, 80)
        cpu.append((k, v))
        dev.append((dk, dv))
    table = hip.ChunkTable([d[0] for d in dev], [d[1] for d in dev])
    out = torch.empty(B, Sq, H, D, dtype=torch.bfloat16, device="cuda")
    lse = torch.empty(B, H, Sq, dtype=torch.float32, device="cuda")
    hip.attn_jobs_fwd(q.cuda(), table, [[0, 1, 2]], [out], [lse])
    torch.cuda.synchronize()
    ref_out, ref_lse = om.chunk_attention(q, torch.cat([c[0] for c in cpu], 1), torch.cat([c[1] for c in cpu], 1))
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all(), "NaN rows behind a chunk leaked"
    assert (out.float().cpu() - ref_out).abs().max().item() <= OUT_TOL
    assert (lse.cpu() - ref_lse).abs().max().item() <= LSE_TOL
