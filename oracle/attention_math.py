"""Closed-form chunk attention and LSE merge (CPU oracle; test infrastructure only).

Reference behaviour restated here:

* ``flash_attn_func(q, k, v, dropout_p=0.0, return_attn_probs=True)`` as called
  at ``core/attention.py:137-143`` and ``:185-191``: non-causal attention of a
  query shard against ONE key/value chunk with ``softmax_scale = D**-0.5``;
  returns ``out`` with the shape/dtype of ``q`` and the natural-log
  ``softmax_lse`` as fp32 ``[B, H, Sq]``.  ``flash_attn==2.7.0.post2`` is a
  third-party dependency that is not vendored in the reference tree, so what is
  restated is its published contract, not its rounding behaviour.
* ``_update_out_and_lse`` (``utils.py:24-40``) and ``update_out_and_lse``
  (``utils.py:42-84``): the sigmoid / logsigmoid form of merging two attention
  states.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import torch
import torch.nn.functional as F


def chunk_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    scale: Optional[float] = None,
    compute_dtype: torch.dtype = torch.float32,
    q_block: int = 1024,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """One KV chunk of non-causal attention.

    q ``[B,Sq,H,D]``, k/v ``[B,Sk,H,D]`` -> (out ``[B,Sq,H,D]`` in
    ``compute_dtype``, lse ``[B,H,Sq]`` in ``compute_dtype``).
    Follows the call at core/attention.py:185-191: ``S = q k^T * D**-0.5``,
    ``lse = log sum exp S`` (natural log), ``out = softmax(S) v``.
    Queries are processed in blocks so the score matrix stays bounded.
    A chunk with ``Sk == 0`` yields ``out = 0`` and ``lse = -inf`` (the neutral
    element of the merge).
    """
    B, Sq, H, D = q.shape
    Sk = k.shape[1]
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    qf = q.to(compute_dtype).permute(0, 2, 1, 3)  # [B,H,Sq,D]
    kf = k.to(compute_dtype).permute(0, 2, 3, 1)  # [B,H,D,Sk]
    vf = v.to(compute_dtype).permute(0, 2, 1, 3)  # [B,H,Sk,D]
    out = torch.empty(B, H, Sq, D, dtype=compute_dtype)
    lse = torch.empty(B, H, Sq, dtype=compute_dtype)
    if Sk == 0:
        out.zero_()
        lse.fill_(-math.inf)
        return out.permute(0, 2, 1, 3).contiguous(), lse
    for s0 in range(0, Sq, q_block):
        s1 = min(Sq, s0 + q_block)
        scores = torch.matmul(qf[:, :, s0:s1], kf) * scale  # [B,H,q,Sk]
        l = torch.logsumexp(scores, dim=-1)
        p = torch.exp(scores - l.unsqueeze(-1))
        out[:, :, s0:s1] = torch.matmul(p, vf)
        lse[:, :, s0:s1] = l
    return out.permute(0, 2, 1, 3).contiguous(), lse


def merge_pair_literal(
    out: torch.Tensor, lse: torch.Tensor, block_out: torch.Tensor, block_lse: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor]:
    """utils.py:24-40 verbatim in meaning.

    out fp32 ``[B,S,H,D]``, lse fp32 ``[B,S,H,1]``, block_out any float dtype
    ``[B,S,H,D]``, block_lse ``[B,H,S]``.
    """
    block_out = block_out.to(torch.float32)  # utils.py:31
    block_lse = block_lse.transpose(-2, -1).unsqueeze(dim=-1)  # utils.py:32
    out = out - torch.sigmoid(block_lse - lse) * (out - block_out)  # utils.py:38
    lse = lse - F.logsigmoid(lse - block_lse)  # utils.py:39
    return out, lse


def update_out_and_lse(
    out: Optional[torch.Tensor],
    lse: Optional[torch.Tensor],
    block_out: torch.Tensor,
    block_lse: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """utils.py:42-84 without the unused ``slice_`` branch.

    Accepts block_lse as ``[B,H,S]`` or ``[B,S,H,1]`` (utils.py:56-58) and the
    running lse in either layout (utils.py:60-61); the first call initialises
    the running state (utils.py:73-77).
    """
    if block_lse is not None and block_lse.shape[-1] == 1:
        block_lse = block_lse.squeeze(-1).transpose(-1, -2)
    if lse is not None and lse.shape[-1] != 1:
        lse = lse.transpose(-2, -1).unsqueeze(dim=-1)
    if out is None:
        out = block_out.to(torch.float32)
        lse = block_lse.transpose(-2, -1).unsqueeze(dim=-1)
        return out, lse
    return merge_pair_literal(out, lse, block_out, block_lse)


def merge_states_closed_form(
    outs: Sequence[torch.Tensor], lses: Sequence[torch.Tensor]
) -> Tuple[torch.Tensor, torch.Tensor]:
    """N-way merge written the textbook way, independent of the sigmoid form.

    outs[i] ``[B,S,H,D]``, lses[i] ``[B,H,S]``.  ``lse = logsumexp_i lse_i``,
    ``out = sum_i exp(lse_i - lse) out_i``.  Returns (out fp32 ``[B,S,H,D]``,
    lse fp32 ``[B,H,S]``).  States whose lse is -inf contribute nothing; if all
    are -inf the result is ``out = 0, lse = -inf``.
    """
    L = torch.stack([l.to(torch.float64) for l in lses], dim=0)  # [n,B,H,S]
    m = L.max(dim=0).values
    m_safe = torch.where(torch.isinf(m), torch.zeros_like(m), m)
    w = torch.exp(L - m_safe)  # -inf -> 0
    den = w.sum(dim=0)
    lse = m_safe + torch.log(den)
    lse = torch.where(den > 0, lse, torch.full_like(lse, -math.inf))
    wn = torch.where(den > 0, w / den.clamp_min(1e-300), torch.zeros_like(w))  # [n,B,H,S]
    acc = torch.zeros_like(outs[0], dtype=torch.float64)
    for i, o in enumerate(outs):
        acc += wn[i].transpose(-2, -1).unsqueeze(-1) * o.to(torch.float64)
    return acc.to(torch.float32), lse.to(torch.float32)


def full_attention(
    q: torch.Tensor, k_chunks: Sequence[torch.Tensor], v_chunks: Sequence[torch.Tensor],
    compute_dtype: torch.dtype = torch.float32,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Attention of q against the concatenation of all chunks (one softmax)."""
    k = torch.cat(list(k_chunks), dim=1)
    v = torch.cat(list(v_chunks), dim=1)
    return chunk_attention(q, k, v, compute_dtype=compute_dtype)


def varlen_chunk_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens_q: Sequence[int],
                           cu_seqlens_kv: Sequence[int]) -> Tuple[torch.Tensor, torch.Tensor]:
    """``flash_attn_varlen_func`` as called at core/attention.py:314-324,366-376, by its
    published contract: packed ``q [total_q,H,D]``, ``k/v [total_k,H,D]``; segment ``i`` of the
    queries attends to segment ``i`` of the keys only.  Returns (out ``[total_q,H,D]``, lse
    ``[H,total_q]``), both fp32.  Query rows outside every segment get out = 0; a segment
    without keys gets out = 0, lse = -inf.  Each segment is the dense closed form."""
    total_q, H, D = q.shape
    out = torch.zeros(total_q, H, D, dtype=torch.float32)
    lse = torch.full((H, total_q), -math.inf, dtype=torch.float32)
    for i in range(len(cu_seqlens_q) - 1):
        q0, q1 = int(cu_seqlens_q[i]), int(cu_seqlens_q[i + 1])
        k0, k1 = int(cu_seqlens_kv[i]), int(cu_seqlens_kv[i + 1])
        if q1 <= q0:
            continue
        o, l = chunk_attention(q[None, q0:q1], k[None, k0:k1], v[None, k0:k1])
        out[q0:q1] = o[0]
        lse[:, q0:q1] = l[0]
    return out, lse


def rel_l1(new: torch.Tensor, ori: torch.Tensor) -> float:
    """utils.py:202-267, tensor branch: ``mean|new-ori| / (mean|ori| + 1e-8)``
    over entries where neither is NaN; ``inf`` if nothing is valid; falls back
    to ``mean|new|`` when ``mean|ori| < 1e-6`` (utils.py:236-238)."""
    valid = ~(torch.isnan(new) | torch.isnan(ori))
    if not bool(valid.any()):
        return float("inf")
    nv = new[valid].to(torch.float32)
    ov = ori[valid].to(torch.float32)
    new_abs_mean = nv.abs().mean().item()
    ori_abs_mean = ov.abs().mean().item()
    if ori_abs_mean < 1e-6:
        return new_abs_mean
    val = (nv - ov).abs().mean().item() / (ori_abs_mean + 1e-8)
    if math.isnan(val) or math.isinf(val):
        return float("inf")
    return val


def bf16_round(x: torch.Tensor) -> torch.Tensor:
    """Round-trip through bf16 (what the HBM state cache does to ``out``)."""
    return x.to(torch.bfloat16).to(torch.float32)
