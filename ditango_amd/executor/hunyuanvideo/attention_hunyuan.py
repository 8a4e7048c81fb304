"""HunyuanVideo attention adapter: ``Hunyuan_DiTangoProcessor`` of executor/hunyuanvideo/attention_hunyuan.py:25-63.

``ringfusion_attn`` takes q / k / v as ``[B,S,H,D]`` with the packed batch's ``cu_seqlens`` (int32 tensors on the
GPU, two segments per sample: valid tokens, padded text; executor/hunyuanvideo/hunyuan_transformer.py:783-792),
flattens them to ``[B*S,H,D]``, runs ``proAttention.varlen_attn`` and returns ``[B, S, H*D]``.  The boundaries stay
on the device (the kernels read them), so the call does not synchronise with the GPU.
"""
from __future__ import annotations

from ...core.attention import proAttention
from ...core.parallel_state import get_isp_group

MEMORY_LAYOUT = {
    "flash": (lambda x: x.view(x.shape[0] * x.shape[1], *x.shape[2:]), lambda x: x),
    "torch": (lambda x: x.transpose(1, 2), lambda x: x.transpose(1, 2)),
    "vanilla": (lambda x: x.transpose(1, 2), lambda x: x.transpose(1, 2)),
    "oAttn": (lambda x: x.view(x.shape[0] * x.shape[1], *x.shape[2:]), lambda x: x),
}


class Hunyuan_DiTangoProcessor:
    def __init__(self, layer_id: int):
        self.oAttn = proAttention(layer_id, get_isp_group())
        self.varlen_Attn = self.oAttn.varlen_attn

    def ringfusion_attn(self, q, k, v, drop_rate=0, attn_mask=None, causal=False, cu_seqlens_q=None, cu_seqlens_kv=None,
                        max_seqlen_q=None, max_seqlen_kv=None, batch_size=1):
        pre_attn_layout, post_attn_layout = MEMORY_LAYOUT["flash"]
        q, k, v = pre_attn_layout(q), pre_attn_layout(k), pre_attn_layout(v)
        x = self.varlen_Attn(q, k, v, cu_seqlens_q, cu_seqlens_kv, max_seqlen_q, max_seqlen_kv)
        x = x.view(batch_size, max_seqlen_q, x.shape[-2], x.shape[-1])   # [b, s, a, d]
        x = post_attn_layout(x)
        b, s, a, d = x.shape
        return x.reshape(b, s, -1)
