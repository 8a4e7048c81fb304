"""Producer side of an attention call: QK normalisation + rotary embedding in one HIP pass.

The reference's executors run these as chains of eager torch ops right before
``proAttention.attn`` / ``varlen_attn``:

* CogVideoX  ``executor/cogvideox/attention_processor.py:55-71``  LayerNorm over D, interleaved RoPE
  on the video tokens only, ``transpose(1, 2).contiguous()``;
* HunyuanVideo  ``executor/hunyuanvideo/hunyuan_transformer.py:177-191``  RMSNorm over D, interleaved RoPE;
* Step-Video  ``executor/step/blocks.py:66-75`` + ``executor/step/rope.py:13-90``  RMSNorm, rotate-half RoPE
  on the sections ``[64, 32, 32]`` of D.

``prepare_qk`` does the whole chain in one launch of ``dt_qk_norm_rope`` and writes the bf16 (or fp16)
``[B,S,H,D]`` tensor the attention kernels read.  There is no non-HIP fallback.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import torch

from . import _hip

_NORMS = {None: _hip.DT_NORM_NONE, "none": _hip.DT_NORM_NONE, "rms": _hip.DT_NORM_RMS,
          "layer_norm": _hip.DT_NORM_LAYER, "layer": _hip.DT_NORM_LAYER}
_ROPES = {None: _hip.DT_ROPE_NONE, "none": _hip.DT_ROPE_NONE, "interleaved": _hip.DT_ROPE_INTERLEAVED,
          "rotate_half": _hip.DT_ROPE_HALVES, "halves": _hip.DT_ROPE_HALVES}


def _f32(t: Optional[torch.Tensor], device) -> Optional[torch.Tensor]:
    if t is None:
        return None
    return t.detach().to(device=device, dtype=torch.float32).contiguous()


def prepare_qk(x: torch.Tensor, *, norm: Optional[str] = None, weight: Optional[torch.Tensor] = None,
               bias: Optional[torch.Tensor] = None, eps: float = 1e-6, rope: Optional[str] = None,
               freqs_cis: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, rope_begin: int = 0,
               rope_end: Optional[int] = None, sections: Sequence[int] = (), match_eager_rounding: bool = False,
               bf16_rope_math: bool = False, out: Optional[torch.Tensor] = None,
               fold_softmax_scale: Optional[float] = None) -> torch.Tensor:
    """x: bf16 (or fp16: a model run in fp16) ``[B,S,H,D]`` view (e.g. a slice of a fused QKV projection; only
    the last dimension must be contiguous).  Returns ``[B,S,H,D]`` contiguous in x's dtype; where "bf16" is said
    below, an fp16 x reads "fp16".

    norm: ``"rms"`` | ``"layer_norm"`` | None, with ``weight`` / ``bias`` of shape ``[D]`` (any float dtype).
    rope: ``"interleaved"`` (pairs ``(2i, 2i+1)``; CogVideoX, HunyuanVideo) | ``"rotate_half"`` (Step-Video,
    per section of ``sections``) | None; ``freqs_cis = (cos, sin)`` of shape ``[rope_end-rope_begin, D]``
    (or with a leading batch dimension), as the callers already hold them; token ``s`` reads row
    ``s - rope_begin``.  ``match_eager_rounding`` rounds to bf16 where the callers' bf16 norm modules do;
    ``bf16_rope_math`` additionally rounds both RoPE products (Step-Video computes RoPE in bf16).

    ``fold_softmax_scale`` (for q only): multiplies the result by ``folded_scale(D, fold_softmax_scale)`` =
    ``softmax_scale * log2(e)`` before the rounding to bf16 (pass 0 for the default ``D ** -0.5``).  The
    attention object must then be told with ``proAttention.q_prescaled = True``: its softmax needs a
    quarter fewer vector instructions.  q differs from the unscaled one by its rounding only, but it is
    not the tensor the reference would hand to ``attn`` -- an opt-in, not part of the drop-in path."""
    if norm not in _NORMS or rope not in _ROPES:
        raise ValueError(f"unknown norm {norm!r} or rope {rope!r}")
    cos = sin = None
    if _ROPES[rope] != _hip.DT_ROPE_NONE:
        if freqs_cis is None:
            raise ValueError("rope needs freqs_cis = (cos, sin)")
        cos, sin = _f32(freqs_cis[0], x.device), _f32(freqs_cis[1], x.device)
    rounding = (_hip.DT_ROUND_NORM_BF16 if match_eager_rounding else 0) | (_hip.DT_ROUND_ROPE_BF16 if bf16_rope_math else 0)
    return _hip.qk_norm_rope(x, norm=_NORMS[norm], weight=_f32(weight, x.device), bias=_f32(bias, x.device), eps=eps,
                             rope=_ROPES[rope], cos=cos, sin=sin, rope_begin=rope_begin, rope_end=rope_end,
                             sections=sections, rounding=rounding, out=out,
                             out_scale=1.0 if fold_softmax_scale is None else folded_scale(x.shape[-1], fold_softmax_scale))


def folded_scale(head_dim: int, softmax_scale: float = 0.0) -> float:
    """``softmax_scale * log2(e)`` (``softmax_scale <= 0``: flash_attn's default ``head_dim ** -0.5``): what a
    caller multiplies q by (before rounding it to bf16) to run the attention with ``q_prescaled``."""
    scale = softmax_scale if softmax_scale and softmax_scale > 0 else head_dim ** -0.5
    return scale * math.log2(math.e)


def rope3d_tables(f: int, h: int, w: int, ch_split: Sequence[int] = (64, 32, 32), dtype: torch.dtype = torch.bfloat16,
                  base: float = 1e4, device=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-token (cos, sin) tables ``[f*h*w, sum(ch_split)]`` fp32 for Step-Video's 3-D RoPE, so that
    ``prepare_qk(..., rope="rotate_half", sections=ch_split, freqs_cis=tables)`` equals
    ``RoPE3D(tokens, (f,h,w), ch_split)`` (executor/step/rope.py:56-90).  Angles are rounded to ``dtype``
    before cos/sin as rope.py:18 does, and cos/sin are evaluated in ``dtype``.  A sequence-parallel rank
    slices the rows of its token shard (rope.py:83-85)."""
    pos = torch.cartesian_prod(torch.arange(f), torch.arange(h), torch.arange(w)).view(-1, 3)
    n_pos = int(pos.max()) + 1
    t = torch.arange(n_pos, dtype=torch.float32)
    cos_parts, sin_parts = [], []
    for i, d in enumerate(ch_split):
        inv = 1.0 / (base ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
        ang = torch.outer(t, inv).to(dtype)
        ang = torch.cat((ang, ang), dim=-1)[pos[:, i]]
        cos_parts.append(ang.cos().to(torch.float32))
        sin_parts.append(ang.sin().to(torch.float32))
    cos, sin = torch.cat(cos_parts, dim=-1).contiguous(), torch.cat(sin_parts, dim=-1).contiguous()
    if device is not None:
        cos, sin = cos.to(device), sin.to(device)
    return cos, sin
