"""QK normalisation and rotary embedding in front of the attention call (CPU oracle; test
infrastructure only).

What the reference's callers do before ``proAttention.attn`` / ``varlen_attn``, restated with
plain torch ops:

* CogVideoX, ``executor/cogvideox/attention_processor.py:55-71``: ``attn.norm_q`` / ``norm_k``
  (diffusers' ``Attention`` with ``qk_norm="layer_norm"``: ``nn.LayerNorm(head_dim)``), then
  ``apply_rotary_emb`` of diffusers 0.31.0 (requirements.txt:2) on the video tokens only
  (``query[:, :, text_seqlen:]``), then ``transpose(1, 2).contiguous()``.
* HunyuanVideo, ``executor/hunyuanvideo/hunyuan_transformer.py:177-191``: ``RMSNorm(head_dim,
  eps=1e-6)`` and ``apply_rotary_emb(..., head_first=False)`` from the ``hyvideo`` package.
* Step-Video, ``executor/step/blocks.py:66-75``: ``RMSNorm(head_dim)`` and ``RoPE3D`` from
  ``executor/step/rope.py:13-90`` with ``rope_ch_split = [64, 32, 32]`` (blocks.py:45).

``diffusers`` and ``hyvideo`` / ``stepvideo`` are third-party packages that are not part of the
reference tree: their published formulas are restated (pairs ``(2i, 2i+1)`` rotate together;
``out = x.float() * cos + rotate(x).float() * sin``, cast back; RMSNorm computes
``x.float() * rsqrt(mean(x^2) + eps)``, casts to the input dtype and multiplies by the
weight), so the exact placement of their intermediate roundings is **parity unpinned**.  The
rotate-half form and the table construction of Step-Video are in the reference's own file
and are followed line by line.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import torch

NORM_NONE, NORM_RMS, NORM_LAYER = 0, 1, 2
ROPE_NONE, ROPE_INTERLEAVED, ROPE_HALVES = 0, 1, 2
ROUND_NORM_BF16, ROUND_ROPE_BF16 = 1, 2


def _r(x: torch.Tensor, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    return x.to(dtype).to(torch.float32)


def _model_dtype(x: torch.Tensor) -> torch.dtype:
    """The dtype the callers' eager modules round to: the activations' own (fp16 for a model run in fp16), bf16
    for anything else."""
    return torch.float16 if x.dtype == torch.float16 else torch.bfloat16


def rms_norm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float, round_bf16: bool,
             round_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """``x.float() * rsqrt(mean(x^2, -1) + eps)`` [cast to the model dtype] ``* weight`` [cast again]; fp32 result."""
    xf = x.to(torch.float32)
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    if round_bf16:
        y = _r(y, round_dtype)
    if weight is not None:
        y = y * weight.to(torch.float32)
        if round_bf16:
            y = _r(y, round_dtype)
    return y


def layer_norm(x: torch.Tensor, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor], eps: float,
               round_bf16: bool, round_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """LayerNorm over the last dimension (biased variance); fp32 math, one rounding at the end if asked."""
    xf = x.to(torch.float32)
    mu = xf.mean(-1, keepdim=True)
    var = (xf - mu).pow(2).mean(-1, keepdim=True)
    y = (xf - mu) * torch.rsqrt(var + eps)
    if weight is not None:
        y = y * weight.to(torch.float32)
    if bias is not None:
        y = y + bias.to(torch.float32)
    return _r(y, round_dtype) if round_bf16 else y


def rotate_interleaved(x: torch.Tensor) -> torch.Tensor:
    """``stack([-x_imag, x_real], -1).flatten`` with ``x_real, x_imag = x.reshape(..., -1, 2).unbind(-1)``."""
    xr, xi = x.reshape(*x.shape[:-1], -1, 2).unbind(-1)
    return torch.stack([-xi, xr], dim=-1).flatten(-2)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """executor/step/rope.py:25-28."""
    x1, x2 = x[..., : x.shape[-1] // 2], x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


def rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, kind: int, sections: Sequence[int] = (),
         bf16_math: bool = False, round_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """x fp32 ``[B,S,H,D]``; cos/sin ``[S,D]`` or ``[B,S,D]``.  fp32 result.

    ``bf16_math`` follows executor/step/rope.py:30-35, where the whole expression
    ``tokens * cos + rotate_half(tokens) * sin`` runs in the tokens' dtype: both products and the
    sum are rounded to that dtype (the sum's rounding is the caller's final cast here)."""
    if cos.dim() == 2:
        cos, sin = cos[None], sin[None]
    cos, sin = cos[:, :, None, :].to(torch.float32), sin[:, :, None, :].to(torch.float32)
    if kind == ROPE_INTERLEAVED:
        rot = rotate_interleaved(x)
    else:
        secs = list(sections) if len(sections) else [x.shape[-1]]
        assert sum(secs) == x.shape[-1]
        rot = torch.cat([rotate_half(p) for p in torch.split(x, secs, dim=-1)], dim=-1)  # rope.py:79-88
    a, b = x * cos, rot * sin
    if bf16_math:
        a, b = _r(a, round_dtype), _r(b, round_dtype)
    return a + b


def qk_norm_rope(x: torch.Tensor, norm: int = NORM_NONE, weight: Optional[torch.Tensor] = None,
                 bias: Optional[torch.Tensor] = None, eps: float = 1e-6, rope_kind: int = ROPE_NONE,
                 cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None, rope_begin: int = 0,
                 rope_end: Optional[int] = None, sections: Sequence[int] = (), rounding: int = 0,
                 out_scale: float = 1.0) -> torch.Tensor:
    """The whole producer step on x ``[B,S,H,D]`` (bf16, or fp16 for a model run in fp16); returns the fp32
    value BEFORE the final rounding to x's dtype (the caller rounds, so a test can bound the distance to the
    exact value).  The intermediate roundings ``rounding`` asks for are to x's dtype.
    ``out_scale`` multiplies the result (fp32) last: a caller's way of folding the softmax scale into q."""
    rn = bool(rounding & ROUND_NORM_BF16)
    rd = _model_dtype(x)
    if norm == NORM_RMS:
        y = rms_norm(x, weight, eps, rn, rd)
    elif norm == NORM_LAYER:
        y = layer_norm(x, weight, bias, eps, rn, rd)
    else:
        y = x.to(torch.float32)
    if rope_kind != ROPE_NONE:
        S = x.shape[1]
        rope_end = S if rope_end is None else rope_end
        if rope_end > rope_begin:
            y = y.clone()
            y[:, rope_begin:rope_end] = rope(y[:, rope_begin:rope_end], cos, sin, rope_kind, sections,
                                             bool(rounding & ROUND_ROPE_BF16), rd)
    if out_scale != 1.0:
        y = y * torch.tensor(out_scale, dtype=torch.float32)
    return y


def rope1d_cos_sin(D: int, seq_len: int, dtype: torch.dtype, base: float = 1e4) -> Tuple[torch.Tensor, torch.Tensor]:
    """executor/step/rope.py:13-23: ``freqs = outer(t, base^(-arange(0,D,2)/D)).to(dtype)``, duplicated
    ``cat((freqs, freqs))``, then cos / sin IN ``dtype``."""
    inv_freq = 1.0 / (base ** (torch.arange(0, D, 2).float() / D))
    t = torch.arange(seq_len, dtype=inv_freq.dtype)
    freqs = torch.einsum("i,j->ij", t, inv_freq).to(dtype)
    freqs = torch.cat((freqs, freqs), dim=-1)
    return freqs.cos(), freqs.sin()


def rope3d_tables(f: int, h: int, w: int, ch_split: Sequence[int], dtype: torch.dtype = torch.bfloat16,
                  base: float = 1e4) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-token tables ``[f*h*w, sum(ch_split)]`` equal to what RoPE3D gathers section by section
    (executor/step/rope.py:56-66, 75-90): token ``n`` of ``cartesian_prod(arange(f), arange(h),
    arange(w))`` uses position ``mesh[n, i]`` in section ``i``; every section's table has
    ``max(mesh) + 1`` rows (rope.py:81)."""
    mesh = torch.cartesian_prod(torch.arange(f), torch.arange(h), torch.arange(w)).view(f * h * w, 3)
    n_pos = int(mesh.max()) + 1
    cs, sn = [], []
    for i, D in enumerate(ch_split):
        c, s = rope1d_cos_sin(D, n_pos, dtype, base)
        cs.append(c[mesh[:, i]])
        sn.append(s[mesh[:, i]])
    return torch.cat(cs, dim=-1), torch.cat(sn, dim=-1)
