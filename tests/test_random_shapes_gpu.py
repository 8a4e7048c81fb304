"""Seeded random shapes through the attention entry points: batch, heads, head dim, query count,
chunk counts and lengths (zero-length chunks included), strided K/V, query and key sub-ranges --
each case against the closed-form oracle (out <= 2e-2, lse <= 1e-3)."""
import random

import pytest
import torch

from oracle import attention_math as om

pytestmark = pytest.mark.gpu

OUT_TOL, LSE_TOL = 2e-2, 1e-3


def _case(rng: random.Random):
    D = rng.choice([64, 128])
    B = rng.choice([1, 1, 2])
    H = rng.choice([1, 2, 3, 5])
    Sq = rng.choice([1, 31, 32, 33, 100, 255, 256, 257, 300, 513])
    C = rng.choice([1, 2, 3, 5])
    lens = [rng.choice([0, 1, 7, 63, 64, 65, 100, 128, 191, 200, 257]) for _ in range(C)]
    if sum(lens) == 0:
        lens[0] = 17
    return D, B, H, Sq, lens


@pytest.mark.parametrize("seed", range(40))
def test_random_jobs(hip, seed):
    rng = random.Random(seed)
    D, B, H, Sq, lens = _case(rng)
    g = torch.Generator().manual_seed(1000 + seed)
    scale_q = rng.choice([0.5, 1.0, 3.0])
    q = (torch.randn(B, Sq, H, D, generator=g) * scale_q).bfloat16()
    # K/V of all chunks cut out of one padded buffer, so chunk rows are strided views
    pad = rng.choice([0, 8, 24])
    kbuf = torch.randn(B, sum(lens) + 1, H, D + pad, generator=g).bfloat16()
    vbuf = torch.randn(B, sum(lens) + 1, H, D + pad, generator=g).bfloat16()
    ks, vs, o = [], [], 0
    for n in lens:
        ks.append(kbuf[:, o:o + n, :, :D])
        vs.append(vbuf[:, o:o + n, :, :D])
        o += n
    print(f"case seed={seed} D={D} B={B} H={H} Sq={Sq} lens={lens} pad={pad}", flush=True)
    dk, dv = kbuf.cuda(), vbuf.cuda()
    dks, dvs, o = [], [], 0
    for n in lens:
        dks.append(dk[:, o:o + n, :, :D])
        dvs.append(dv[:, o:o + n, :, :D])
        o += n
    table = hip.ChunkTable(dks, dvs)
    # job 0: every chunk; job 1: one random non-empty chunk; job 2: a query sub-range against key sub-ranges
    nz = [c for c, n in enumerate(lens) if n > 0]
    one = rng.choice(nz)
    qb = rng.randrange(0, Sq)
    ql = rng.randrange(1, Sq - qb + 1)
    sub = []
    for c in nz[:2]:
        kb = rng.randrange(0, lens[c])
        kl = rng.randrange(0, lens[c] - kb + 1)
        sub.append((c, kb, kl))
    jobs = [list(range(len(lens))), [one], [c for c, _, _ in sub]]
    outs = [torch.full((B, Sq, H, D), 9.0, dtype=torch.bfloat16, device="cuda") for _ in jobs]
    lses = [torch.full((B, H, Sq), 9.0, dtype=torch.float32, device="cuda") for _ in jobs]
    q_ranges = [(0, Sq), (0, Sq), (qb, ql)]
    kv_ranges = [[(0, n) for n in lens], [(0, lens[one])], [(kb, kl) for _, kb, kl in sub]]
    hip.attn_jobs_fwd(q.cuda(), table, jobs, outs, lses, q_ranges=q_ranges, kv_ranges=kv_ranges)
    torch.cuda.synchronize()

    def check(j, ref_out, ref_lse, rows=slice(None)):
        out, lse = outs[j].float().cpu()[:, rows], lses[j].cpu()[:, :, rows]
        finite = torch.isfinite(ref_lse)
        assert torch.equal(torch.isfinite(lse), finite)
        err = (out - ref_out).abs().max().item()
        lerr = (lse[finite] - ref_lse[finite]).abs().max().item() if finite.any() else 0.0
        assert err <= OUT_TOL and lerr <= LSE_TOL, f"job {j}: out {err:.3e} lse {lerr:.3e}"

    check(0, *om.full_attention(q, ks, vs))
    check(1, *om.chunk_attention(q, ks[one], vs[one]))
    sk = [ks[c][:, kb:kb + kl] for c, kb, kl in sub]
    sv = [vs[c][:, kb:kb + kl] for c, kb, kl in sub]
    check(2, *om.full_attention(q[:, qb:qb + ql], sk, sv), rows=slice(qb, qb + ql))
    # rows outside the query range of job 2 were left untouched
    mask = torch.ones(Sq, dtype=torch.bool)
    mask[qb:qb + ql] = False
    assert (outs[2].float().cpu()[:, mask] == 9.0).all() and (lses[2].cpu()[:, :, mask] == 9.0).all()
