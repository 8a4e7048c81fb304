"""One-GPU stand-in for the reference's process groups (core/parallel_state.py,
core/group_coordinate.py).

One GPU plays ONE sequence-parallel rank: it owns the local query shard and can
see all ``N`` key/value chunks the ring would deliver.  ``LocalRingGroup``
exposes what the hot path reads from a ``GroupCoordinator`` --
``world_size`` and ``rank_in_group`` (core/attention.py:23,25) -- and replaces
the batched isend/irecv of K/V (core/group_coordinate.py:643-668) by a lookup:
``kv_chunk(c)`` is the K/V the ring would have handed over for chunk ``c``.
"""
from typing import Dict, List, Optional, Sequence, Tuple

import torch


class LocalRingGroup:
    def __init__(self, world_size: int, rank_in_group: int = 0, name: str = "isp"):
        assert world_size >= 1 and 0 <= rank_in_group < world_size
        self.world_size = world_size
        self.rank_in_group = rank_in_group
        self.rank = rank_in_group
        self.ranks = list(range(world_size))
        self.name = name
        self._k: List[Optional[torch.Tensor]] = [None] * world_size
        self._v: List[Optional[torch.Tensor]] = [None] * world_size
        self._cu: List[Optional[Sequence[int]]] = [None] * world_size

    def set_kv_chunks(self, k_chunks: Sequence[torch.Tensor], v_chunks: Sequence[torch.Tensor],
                      cu_seqlens_kv: Optional[Sequence] = None) -> None:
        """K/V of every ring position for the coming attention call ([B,Sk_c,H,D] each, or packed
        [total_c,H,D] for the variable-length entry).  The entry at ``rank_in_group`` may be
        None: the local chunk is the (key, value) passed to ``attn`` itself.
        ``cu_seqlens_kv[c]`` are the segment boundaries of chunk ``c`` (they travel with K/V on
        the reference's ring, core/attention.py:307-311): int32 device tensors as the reference's
        callers make them (hunyuan_transformer.py:789-792) are kept as they are -- nothing is copied to
        the host -- and lists / CPU tensors as lists of ints."""
        assert len(k_chunks) == self.world_size and len(v_chunks) == self.world_size
        self._k = list(k_chunks)
        self._v = list(v_chunks)
        if cu_seqlens_kv is not None:
            assert len(cu_seqlens_kv) == self.world_size
            self._cu = [c if c is None or (torch.is_tensor(c) and c.is_cuda)
                        else [int(x) for x in (c.tolist() if hasattr(c, "tolist") else c)]
                        for c in cu_seqlens_kv]
        else:
            self._cu = [None] * self.world_size

    def kv_cu_seqlens(self, chunk_id: int):
        """Segment boundaries of chunk ``chunk_id``: a list of ints, or the int32 device tensor that was handed in."""
        cu = self._cu[chunk_id]
        if cu is None:
            raise RuntimeError(f"segment boundaries of KV chunk {chunk_id} were not provided (set_kv_chunks)")
        return cu

    def kv_chunk(self, chunk_id: int) -> Tuple[torch.Tensor, torch.Tensor]:
        k, v = self._k[chunk_id], self._v[chunk_id]
        if k is None or v is None:
            raise RuntimeError(f"KV chunk {chunk_id} was not provided to the ring group (set_kv_chunks)")
        return k, v

    def _no_p2p(self, *a, **kw):
        raise NotImplementedError(
            "on one GPU the K/V exchange of the ring is a chunk lookup (LocalRingGroup.kv_chunk); "
            "there is no peer to send to")

    p2p_isend = p2p_irecv = p2p_commit = p2p_wait = _no_p2p


_USP: Optional[LocalRingGroup] = None
_ISP: Dict[int, LocalRingGroup] = {}


def init_local_groups(world_size: int, rank: int = 0) -> LocalRingGroup:
    """Create the USP group (and the ISP group of the same size, which is what
    ``sparse_type='full'`` yields in core/initialize.py:28,46-49)."""
    global _USP
    _USP = LocalRingGroup(world_size, rank, name="usp")
    _ISP.clear()
    _ISP[world_size] = _USP
    return _USP


def destroy_local_groups() -> None:
    global _USP
    _USP = None
    _ISP.clear()


def get_usp_group() -> LocalRingGroup:
    assert _USP is not None, "USP group is not initialized (init_local_groups)"
    return _USP


def get_isp_group(stride: Optional[int] = None) -> LocalRingGroup:
    assert _USP is not None, "ISP group is not initialized (init_local_groups)"
    return _USP


def get_world_group() -> LocalRingGroup:
    return get_usp_group()
