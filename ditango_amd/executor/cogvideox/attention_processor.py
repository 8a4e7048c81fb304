"""CogVideoX attention adapter: ``CVX_oCacheAttnProcessor`` of executor/cogvideox/attention_processor.py:27-86.

Same constructor, same ``__call__`` signature, same result (``hidden_states, encoder_hidden_states``); the
``attn`` argument is diffusers' ``Attention`` module or anything with its fields (``to_q / to_k / to_v``,
``norm_q / norm_k`` = ``nn.LayerNorm(head_dim)`` or None, ``heads``, ``to_out``, ``is_cross_attention``).

What differs from the reference is how the stretch between the projections and the attention runs.  The
reference transposes to ``[B,H,S,D]``, applies the norm modules and ``apply_rotary_emb`` as eager ops on the
video tokens, and transposes back with ``.contiguous()`` (:48-71) -- six passes over q and k.  Here the
projection output is viewed as ``[B,S,H,D]`` (what the kernels read; no transposition at all) and LayerNorm +
RoPE on the rows behind the text tokens are ONE pass each for q and k (``dt_qk_norm_rope``); the attention
writes the activation dtype directly (``proAttention.out_dtype``), so the cast of :80 is no pass either.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from ...core.attention import proAttention
from ...core.parallel_state import get_isp_group
from ...core.redundancy_map import get_redundancy_map
from ...logger import init_logger
from ...producer import prepare_qk

logger = init_logger(__name__)


class CVX_oCacheAttnProcessor:
    def __init__(self, layer_id: int):
        self.oAttn = proAttention(layer_id, get_isp_group())

    @staticmethod
    def _norm_args(norm) -> dict:
        if norm is None:
            return dict(norm=None)
        if not isinstance(norm, torch.nn.LayerNorm):
            raise TypeError(f"norm_q / norm_k must be nn.LayerNorm over the head dimension or None, got {type(norm).__name__}")
        return dict(norm="layer_norm", weight=norm.weight, bias=norm.bias, eps=norm.eps)

    def project_qkv(self, attn, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor,
                    image_rotary_emb: Optional[Tuple[torch.Tensor, torch.Tensor]] = None):
        """(query, key, value) of this rank's token shard, text tokens first, as ``[B,S,H,D]`` (bf16 or fp16, the model's dtype) in the layout
        the attention reads (:39-71 of the reference, without its transposes).  Also what a test or a ring
        stand-in calls to produce the K/V another rank would send."""
        text_seqlen = encoder_hidden_states.size(1)
        batch_size = hidden_states.shape[0]
        x = torch.cat([encoder_hidden_states, hidden_states], dim=1)
        if x.dtype not in (torch.bfloat16, torch.float16):
            raise TypeError(f"the adapter runs bf16 or fp16 activations (the model's dtype), got {x.dtype}")
        query, key, value = attn.to_q(x), attn.to_k(x), attn.to_v(x)
        head_num = attn.heads
        head_dim = key.shape[-1] // head_num
        query = query.view(batch_size, -1, head_num, head_dim)
        key = key.view(batch_size, -1, head_num, head_dim)
        value = value.view(batch_size, -1, head_num, head_dim)
        rope = dict(rope="interleaved", freqs_cis=image_rotary_emb, rope_begin=text_seqlen) if image_rotary_emb is not None else {}
        k_rope = rope if not getattr(attn, "is_cross_attention", False) else {}
        # rounded where the reference's modules round in the model's dtype: after the norm, after the rotation
        query = prepare_qk(query, **self._norm_args(getattr(attn, "norm_q", None)), match_eager_rounding=True, **rope)
        key = prepare_qk(key, **self._norm_args(getattr(attn, "norm_k", None)), match_eager_rounding=True, **k_rope)
        return query, key, value.contiguous()

    def __call__(self, attn, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor,
                 attention_mask: Optional[torch.Tensor] = None,
                 image_rotary_emb: Optional[Tuple[torch.Tensor, torch.Tensor]] = None):
        text_seqlen = encoder_hidden_states.size(1)
        latent_seqlen = hidden_states.size(1)
        batch_size = hidden_states.shape[0]
        assert attention_mask is None
        dtype = hidden_states.dtype
        query, key, value = self.project_qkv(attn, hidden_states, encoder_hidden_states, image_rotary_emb)
        head_num, head_dim = query.shape[2], query.shape[3]
        # the merge writes the activation dtype, so the cast of :80 is no separate pass -- except while the redundancy
        # map is being profiled, whose metric is defined on the fp32 result (core/redundancy_map.py:174-197)
        rm = get_redundancy_map()
        self.oAttn.out_dtype = torch.float32 if (rm is not None and rm.auto_setting) else dtype
        out = self.oAttn.attn(query, key, value)
        out = out.to(dtype)
        hidden_states = out.reshape(batch_size, -1, head_num * head_dim)
        hidden_states = attn.to_out[0](hidden_states)   # linear proj
        hidden_states = attn.to_out[1](hidden_states)   # dropout
        encoder_hidden_states, hidden_states = hidden_states.split([text_seqlen, latent_seqlen], dim=1)
        return hidden_states, encoder_hidden_states
