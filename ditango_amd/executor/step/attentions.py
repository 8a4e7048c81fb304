"""Step-Video-T2V attention adapter: the ``o_attn_func`` path of ``Attention`` in executor/step/attentions.py:23-100.

``attn_processor`` hands out ``o_attn_func`` (the cached block attention) for every attention type but
``'torch'`` and ``'parallel'``; those two and the DistriFusion path (``use_distrifusion``) are the reference's
comparison baselines (scaled_dot_product_attention, xDiT, stale-KV all-gather) and are not part of this package.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from ...core.attention import proAttention
from ...core.config import get_config
from ...core.parallel_state import get_isp_group
from ...core.redundancy_map import get_redundancy_map


class Attention(nn.Module):
    def __init__(self, layer_id: int = -1):
        super().__init__()
        self.config = get_config()
        self.layer_id = layer_id
        if getattr(self.config, "use_distrifusion", False):
            raise NotImplementedError("the DistriFusion baseline (stale K/V all-gather) is not part of this package")
        self.oAttn = proAttention(layer_id, get_isp_group())

    def attn_processor(self, attn_type):
        if attn_type in ("torch", "parallel"):
            raise NotImplementedError(f"attention type {attn_type!r} is one of the reference's comparison baselines, "
                                      "not the cached block attention")
        return self.o_attn_func

    def o_attn_func(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, causal: bool = False, **kwargs) -> torch.Tensor:
        """q / k / v ``[B,S,H,D]`` of this rank's shard -> ``[B,S,H,D]`` in q's dtype (:85-100).  The merge kernel
        writes that dtype itself; the reference's ``.to(q.dtype)`` pass disappears."""
        rm = get_redundancy_map()
        profiling = rm is not None and rm.auto_setting      # the profiled metric is defined on the fp32 result
        self.oAttn.out_dtype = q.dtype if (q.dtype in (torch.bfloat16, torch.float16) and not profiling) else torch.float32
        x = self.oAttn.attn(q, k, v)
        return x.to(q.dtype)
