"""Helpers of the hot path with the reference's names (utils.py): the global
diffusion-step counter, the LSE merge and the relative-L1 metric.  The merge and
the metric run in HIP kernels (``dt_merge_states``, ``dt_rel_l1_sums``)."""
import math
from typing import Dict, List, Optional, Tuple

import torch

from . import _hip
from .logger import init_logger

logger = init_logger(__name__)

_PADDING_DICT: Dict[str, List[int]] = {}
_TIMESTEP: int = 0


def get_timestep() -> int:
    return _TIMESTEP


def update_timestep(timestep: int) -> None:
    global _TIMESTEP
    _TIMESTEP = timestep


def update_out_and_lse(out: Optional[torch.Tensor], lse: Optional[torch.Tensor],
                       block_out: torch.Tensor, block_lse: torch.Tensor, slice_=None
                       ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Drop-in for utils.py:42-84.

    Merges the state ``(block_out, block_lse)`` into the running state and returns
    the running state as (fp32 ``[B,S,H,D]``, fp32 ``[B,S,H,1]``).  ``block_lse``
    may be ``[B,H,S]`` or ``[B,S,H,1]``, the running ``lse`` either layout
    (utils.py:56-61).  One fused kernel pass instead of the reference's chain of
    elementwise ops; the result is a new tensor (the reference is out-of-place too).
    """
    if slice_ is not None:
        if out is None:
            raise RuntimeError("first update_out_and_lse should not pass slice_ args")
        s_out, s_lse = update_out_and_lse(out[slice_].contiguous(), lse[slice_].contiguous(), block_out, block_lse)
        out[slice_], lse[slice_] = s_out, s_lse
        return out, lse
    block_out = block_out.contiguous()
    if out is None:
        return _hip.merge_states([block_out], [block_lse], dst_dtype=torch.float32, dst_lse_bsh=True)
    return _hip.merge_states([out.contiguous(), block_out], [lse, block_lse], dst_dtype=torch.float32, dst_lse_bsh=True)


def _update_out_and_lse(out: torch.Tensor, lse: torch.Tensor, block_out: torch.Tensor, block_lse: torch.Tensor
                        ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Drop-in for utils.py:24-40: the two-state merge on an existing running state (fp32 ``out``
    ``[B,S,H,D]``, fp32 ``lse [B,S,H,1]``; ``block_lse`` in flash-attn's ``[B,H,S]``).  One
    ``dt_merge_states`` launch with n = 2."""
    return _hip.merge_states([out.contiguous(), block_out.contiguous()], [lse, block_lse], dst_dtype=torch.float32,
                             dst_lse_bsh=True)


def rel_l1(new, ori) -> float:
    """Drop-in for utils.py:202-267.  Tensor inputs are reduced on the GPU in one
    kernel and read back once (the reference syncs three times)."""
    if torch.is_tensor(new) and torch.is_tensor(ori):
        a = new.to(torch.float32).contiguous()
        b = ori.to(torch.float32).contiguous()
        s = _hip.rel_l1_sums(a, b).cpu()
        cnt = s[3].item()
        if cnt == 0:
            print("WARNING: All values are NaN in tensors")
            return float("inf")
        new_abs_mean = s[1].item() / cnt
        ori_abs_mean = s[2].item() / cnt
        if ori_abs_mean < 1e-6:
            print(f"WARNING: Reference magnitude is very small ({ori_abs_mean}), using absolute difference")
            return new_abs_mean
        val = (s[0].item() / cnt) / (ori_abs_mean + 1e-8)
    else:
        if (isinstance(new, float) and math.isnan(new)) or (isinstance(ori, float) and math.isnan(ori)):
            print("WARNING: NaN detected in scalar inputs")
            return float("inf")
        if abs(ori) < 1e-6:
            print(f"WARNING: Reference magnitude is very small ({abs(ori)}), using absolute value")
            return abs(new)
        val = abs(new - ori) / (abs(ori) + 1e-8)
    if isinstance(val, float) and (math.isnan(val) or math.isinf(val)):
        print(f"WARNING: Invalid result ({val}) in rel_l1 calculation")
        return float("inf")
    return val


def split_tensor_uneven(tensor: torch.Tensor, world_size: int, dim: int = 1,
                        tensor_name: Optional[str] = None) -> List[torch.Tensor]:
    """utils.py:86-136: split into ``world_size`` shards of equal length, the first
    ``len % world_size`` shards one token longer, the rest zero-padded to match."""
    seq_len = tensor.shape[dim]
    base, rem = divmod(seq_len, world_size)
    target = base + (1 if rem > 0 else 0)
    splits, pads, start = [], [], 0
    for i in range(world_size):
        length = base + (1 if i < rem else 0)
        part = tensor.narrow(dim, start, length)
        pad = target - length
        pads.append(pad)
        if pad > 0:
            shape = list(part.shape)
            shape[dim] = pad
            part = torch.cat([part, torch.zeros(shape, dtype=part.dtype, device=part.device)], dim=dim)
        splits.append(part)
        start += length
    if tensor_name is not None:
        _PADDING_DICT[tensor_name] = pads
    return splits


def get_padding_dict() -> Dict[str, List[int]]:
    return _PADDING_DICT


def remove_padding_after_gather(tensor: torch.Tensor, tensor_name: str) -> torch.Tensor:
    """utils.py:142-167."""
    if tensor_name not in _PADDING_DICT:
        return tensor
    pads = _PADDING_DICT[tensor_name]
    seg = tensor.size(1) // len(pads)
    idx: List[int] = []
    for r, pad in enumerate(pads):
        idx.extend(range(r * seg, r * seg + seg - pad))
    return tensor.index_select(1, torch.tensor(idx, device=tensor.device))
