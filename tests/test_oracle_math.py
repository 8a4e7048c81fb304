"""Pins the arithmetic of the CPU oracle against library routines and identities
(nothing here retypes the oracle's own formula)."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import attention_math as om


def _rand(B, Sq, Sk, H, D, seed, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(B, Sq, H, D, generator=g, dtype=dtype), torch.randn(B, Sk, H, D, generator=g, dtype=dtype),
            torch.randn(B, Sk, H, D, generator=g, dtype=dtype))


@pytest.mark.parametrize("B,Sq,Sk,H,D", [(1, 7, 5, 1, 8), (2, 33, 70, 3, 64), (1, 130, 257, 2, 128)])
def test_chunk_attention_vs_sdpa_and_logsumexp(B, Sq, Sk, H, D):
    q, k, v = _rand(B, Sq, Sk, H, D, 1)
    out, lse = om.chunk_attention(q, k, v, compute_dtype=torch.float64, q_block=16)
    ref = F.scaled_dot_product_attention(q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3), v.permute(0, 2, 1, 3))
    assert torch.allclose(out, ref.permute(0, 2, 1, 3), atol=1e-12)
    # lse by brute force, natural log, scale D^-0.5, layout [B,H,Sq]
    for b in range(B):
        for h in range(H):
            s = (q[b, :, h] @ k[b, :, h].T) / math.sqrt(D)
            assert torch.allclose(lse[b, h], torch.logsumexp(s, dim=-1), atol=1e-12)
    assert lse.shape == (B, H, Sq) and out.shape == (B, Sq, H, D)


def test_chunk_attention_special_cases():
    q, k, v = _rand(1, 9, 6, 2, 16, 2)
    # a single key: softmax weight 1 -> out == v, lse == the score
    out, lse = om.chunk_attention(q, k[:, :1], v[:, :1], compute_dtype=torch.float64)
    assert torch.allclose(out, v[:, :1].expand_as(out), atol=1e-12)
    assert torch.allclose(lse, torch.einsum("bshd,bhd->bhs", q, k[:, 0]) / 4.0, atol=1e-12)
    # identical keys: uniform weights -> out == mean(v), lse == score + log(n)
    kk = k[:, :1].expand(-1, 6, -1, -1)
    out, lse2 = om.chunk_attention(q, kk, v, compute_dtype=torch.float64)
    assert torch.allclose(out, v.mean(1, keepdim=True).expand_as(out), atol=1e-12)
    assert torch.allclose(lse2, lse + math.log(6), atol=1e-12)
    # key permutation invariance
    perm = torch.randperm(6, generator=torch.Generator().manual_seed(0))
    o1, l1 = om.chunk_attention(q, k, v, compute_dtype=torch.float64)
    o2, l2 = om.chunk_attention(q, k[:, perm], v[:, perm], compute_dtype=torch.float64)
    assert torch.allclose(o1, o2, atol=1e-12) and torch.allclose(l1, l2, atol=1e-12)
    # empty chunk is the neutral state
    o0, l0 = om.chunk_attention(q, k[:, :0], v[:, :0])
    assert (o0 == 0).all() and torch.isinf(l0).all() and (l0 < 0).all()


@pytest.mark.parametrize("lens", [[5, 9], [16, 1, 30, 7], [3, 0, 11]])
def test_full_attention_equals_merge_of_chunks(lens):
    B, Sq, H, D = 2, 21, 3, 32
    g = torch.Generator().manual_seed(4)
    q = torch.randn(B, Sq, H, D, generator=g, dtype=torch.float64)
    ks = [torch.randn(B, n, H, D, generator=g, dtype=torch.float64) for n in lens]
    vs = [torch.randn(B, n, H, D, generator=g, dtype=torch.float64) for n in lens]
    full_out, full_lse = om.full_attention(q, ks, vs, compute_dtype=torch.float64)
    states = [om.chunk_attention(q, k, v, compute_dtype=torch.float64) for k, v in zip(ks, vs)]
    # closed-form N-way merge
    m_out, m_lse = om.merge_states_closed_form([s[0] for s in states], [s[1] for s in states])
    assert torch.allclose(m_out.double(), full_out, atol=1e-6) and torch.allclose(m_lse.double(), full_lse, atol=1e-6)
    # literal sigmoid/logsigmoid fold (fp32 like the reference) in two different orders
    for order in (range(len(lens)), reversed(range(len(lens)))):
        o = l = None
        for i in order:
            if lens[i] == 0:
                continue  # the reference never merges an absent state
            o, l = om.update_out_and_lse(o, l, states[i][0].float(), states[i][1].float())
        assert torch.allclose(o.double(), full_out, atol=1e-5)
        assert torch.allclose(l.squeeze(-1).transpose(1, 2).double(), full_lse, atol=1e-5)


def test_merge_pair_is_logaddexp_and_weighted_average():
    g = torch.Generator().manual_seed(6)
    B, S, H, D = 1, 13, 2, 8
    o1, o2 = torch.randn(B, S, H, D, generator=g), torch.randn(B, S, H, D, generator=g)
    l1, l2 = torch.randn(B, H, S, generator=g) * 4, torch.randn(B, H, S, generator=g) * 4
    out, lse = om.merge_pair_literal(o1, l1.transpose(1, 2).unsqueeze(-1), o2, l2)
    ref_lse = torch.logaddexp(l1, l2)
    w1 = torch.exp(l1 - ref_lse).transpose(1, 2).unsqueeze(-1)
    w2 = torch.exp(l2 - ref_lse).transpose(1, 2).unsqueeze(-1)
    assert torch.allclose(lse.squeeze(-1).transpose(1, 2), ref_lse, atol=1e-5)
    assert torch.allclose(out, w1 * o1 + w2 * o2, atol=1e-5)
    # commutative
    out_b, lse_b = om.merge_pair_literal(o2, l2.transpose(1, 2).unsqueeze(-1), o1, l1)
    assert torch.allclose(out, out_b, atol=1e-5) and torch.allclose(lse, lse_b, atol=1e-5)
    # merging an empty state (-inf) changes nothing
    out_c, lse_c = om.merge_pair_literal(o1, l1.transpose(1, 2).unsqueeze(-1), o2, torch.full_like(l2, -math.inf))
    assert torch.equal(out_c, o1) and torch.equal(lse_c, l1.transpose(1, 2).unsqueeze(-1))


def test_update_out_and_lse_layouts():
    g = torch.Generator().manual_seed(8)
    B, S, H, D = 2, 5, 3, 4
    o1, o2 = torch.randn(B, S, H, D, generator=g), torch.randn(B, S, H, D, generator=g)
    l1, l2 = torch.randn(B, H, S, generator=g), torch.randn(B, H, S, generator=g)
    a_out, a_lse = om.update_out_and_lse(None, None, o1.bfloat16(), l1)
    assert a_out.dtype == torch.float32 and a_lse.shape == (B, S, H, 1)
    r1 = om.update_out_and_lse(a_out, a_lse, o2, l2)
    r2 = om.update_out_and_lse(a_out, a_lse.squeeze(-1).transpose(1, 2), o2, l2.transpose(1, 2).unsqueeze(-1))
    assert torch.equal(r1[0], r2[0]) and torch.equal(r1[1], r2[1])


def test_rel_l1_closed_form():
    a = torch.tensor([1.0, -2.0, float("nan"), 4.0])
    b = torch.tensor([1.5, -2.0, 3.0, float("nan")])
    # valid entries: (1,1.5), (-2,-2): mean|a-b| = 0.25, mean|b| = 1.75
    assert abs(om.rel_l1(a, b) - 0.25 / (1.75 + 1e-8)) < 1e-7
    assert om.rel_l1(torch.tensor([float("nan")]), torch.tensor([1.0])) == float("inf")
    assert om.rel_l1(torch.tensor([3.0, -5.0]), torch.tensor([0.0, 0.0])) == 4.0


def test_varlen_attention_is_block_diagonal_attention():
    g = torch.Generator().manual_seed(12)
    q = torch.randn(20, 2, 16, generator=g)
    k = torch.randn(30, 2, 16, generator=g)
    v = torch.randn(30, 2, 16, generator=g)
    # one segment spanning everything is the dense call
    o, l = om.varlen_chunk_attention(q, k, v, [0, 20], [0, 30])
    od, ld = om.chunk_attention(q[None], k[None], v[None])
    assert torch.equal(o, od[0]) and torch.equal(l, ld[0])
    # two segments == attention under a block-diagonal mask (library routine)
    o, l = om.varlen_chunk_attention(q, k, v, [0, 12, 20], [0, 25, 30])
    mask = torch.zeros(20, 30, dtype=torch.bool)
    mask[:12, :25] = True
    mask[12:, 25:] = True
    ref = F.scaled_dot_product_attention(q.permute(1, 0, 2)[None], k.permute(1, 0, 2)[None], v.permute(1, 0, 2)[None],
                                         attn_mask=mask)[0].permute(1, 0, 2)
    assert torch.allclose(o, ref, atol=1e-5)
    # a segment without keys is the neutral state; rows outside every segment stay zero
    o, l = om.varlen_chunk_attention(q, k, v, [0, 12, 18], [0, 30, 30])
    assert (o[12:] == 0).all() and torch.isinf(l[:, 12:]).all()
