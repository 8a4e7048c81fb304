"""HBM-resident cache of attention states, one per transformer layer.

API of the reference's ``proCache`` (core/cache.py:9-128).  A cached state is
``(out bf16 [B,Sq,H,D] -- fp16 for a model run in fp16 --, lse fp32 [B,H,Sq])`` in device memory -- half the bytes
of the fp32 states the reference keeps -- written by the attention kernel itself
and read exactly once per reuse by the fused merge kernel.

Two storage forms:

* block lists (``out_block_cache`` / ``lse_block_cache``, indexed by block id as
  in the reference) for the stride mode; coarsening to fewer blocks
  (``_merge_blocks``) is one fused merge launch per new block, written in place;
* a contiguous arena ``[C, B, Sq, H, D]`` / ``[C, B, H, Sq]`` plus one scratch
  state for the mask mode, addressed by chunk id from device-side schedules.
"""
from __future__ import annotations

from typing import Callable, List, Optional, Tuple

import torch

from .. import _hip
from ..logger import init_logger
from ..utils import get_timestep

logger = init_logger(__name__)


class proCache:
    def __init__(self, isp_size: int, layer_id: int):
        self.isp_size = isp_size
        self.curr_isp_stride = isp_size
        self.curr_block_num = isp_size
        self.layer_id = layer_id
        self.out_block_cache: List[Optional[torch.Tensor]] = [None] * self.curr_block_num
        self.lse_block_cache: List[Optional[torch.Tensor]] = [None] * self.curr_block_num
        self.full_out_cache = [None]
        self.block_size_mb: Optional[float] = None
        self._memory_constraint: Optional[float] = None
        # injectable probes (MB): current allocation and the budget (0.72 of device memory, cache.py:22)
        self.memory_probe: Callable[[], float] = lambda: torch.cuda.memory_allocated() / (1024 * 1024)
        # mask-mode arena
        self.arena_out: Optional[torch.Tensor] = None
        self.arena_lse: Optional[torch.Tensor] = None
        self.diag_out: Optional[torch.Tensor] = None
        self.diag_lse: Optional[torch.Tensor] = None
        self.arena_valid: List[bool] = []
        self.arena_refused: Optional[tuple] = None  # arena shape the memory guard turned down

    # ---- memory guard (cache.py:89-128) -------------------------------------------------------
    @property
    def memory_constraint(self) -> float:
        if self._memory_constraint is None:
            self._memory_constraint = 0.72 * torch.cuda.get_device_properties(0).total_memory / (1024 * 1024)
        return self._memory_constraint

    @memory_constraint.setter
    def memory_constraint(self, mb: float) -> None:
        self._memory_constraint = mb

    def get_curr_isp_stride(self, layer_id: int) -> int:
        """Stride of the current (step, layer).  The reference's method of this name (core/cache.py:24-26)
        indexes the RedundancyMap object, which has no ``__getitem__``: nothing calls it there.  Here it
        returns what the attention call itself asks the map for (core/attention.py:90)."""
        from .redundancy_map import get_redundancy_map
        return int(get_redundancy_map().get_curr_isp_stride(get_timestep(), layer_id))

    def set_block_size_mb(self, tensor: torch.Tensor) -> float:
        """Size of one cached state for a K/V shard shaped like ``tensor`` ``[B,S,H,D]``:
        bf16 ``out`` plus fp32 ``lse`` = ``(2D + 4)`` bytes per (token, head).  (The
        reference sizes an fp32 ``[..., D+1]`` tensor by allocating it, cache.py:89-101.)"""
        if self.block_size_mb is None:
            rows = tensor.numel() // tensor.shape[-1]
            self.block_size_mb = rows * (2 * tensor.shape[-1] + 4) / (1024 ** 2)
        return self.block_size_mb

    def pass_memory_check(self, next_isp_stride: int, layer_id: int) -> bool:
        """cache.py:103-128"""
        if next_isp_stride == self.isp_size:
            return True
        active = 0
        for i, block in enumerate(self.out_block_cache):
            if block is not None:
                active += 1
                if self.block_size_mb is None and torch.is_tensor(block):  # (dry runs keep chunk-id tuples)
                    mb = block.element_size() * block.nelement() / (1024 ** 2)
                    if self.lse_block_cache[i] is not None:
                        mb += self.lse_block_cache[i].element_size() * self.lse_block_cache[i].nelement() / (1024 ** 2)
                    self.block_size_mb = mb
        if self.block_size_mb is None:
            return True
        predicted = self.isp_size // next_isp_stride
        if predicted <= active:
            return True
        add = self.block_size_mb * (predicted - active)
        now = self.memory_probe()
        if now + add > self.memory_constraint:
            logger.warning(f"T{get_timestep()}L{layer_id} | Memory check failed: {now + add} > {self.memory_constraint}, "
                           f"setting stride {next_isp_stride} to {self.isp_size}")
            return False
        return True

    # ---- block store (cache.py:28-84) -----------------------------------------------------------
    def _merge_blocks(self, new_block_num: int) -> None:
        """Coarsen to ``new_block_num`` blocks: each new block is the LSE merge of
        ``curr/new`` consecutive old ones, empty ones skipped (cache.py:28-46).  One
        fused merge launch per new block with two or more members, written in place
        over its first member; a single member is re-linked without touching memory."""
        assert self.curr_block_num % new_block_num == 0, f"Invalid block number {new_block_num} for merging."
        group = self.curr_block_num // new_block_num
        new_out: List[Optional[torch.Tensor]] = [None] * new_block_num
        new_lse: List[Optional[torch.Tensor]] = [None] * new_block_num
        for i in range(new_block_num):
            outs, lses = [], []
            for j in range(group):
                o = self.out_block_cache[i * group + j]
                l = self.lse_block_cache[i * group + j]
                if l is not None:
                    outs.append(o)
                    lses.append(l)
            if len(outs) == 1:
                new_out[i], new_lse[i] = outs[0], lses[0]
            elif len(outs) > 1:
                _hip.merge_states(outs, lses, dst_out=outs[0], dst_lse=lses[0])
                new_out[i], new_lse[i] = outs[0], lses[0]
        self.out_block_cache = new_out
        self.lse_block_cache = new_lse

    def update_cache_blocks(self, new_isp_stride: int, next_target_block_id: int) -> None:
        """cache.py:49-72"""
        if new_isp_stride == self.isp_size:
            self.curr_isp_stride = self.isp_size
            self.curr_block_num = self.isp_size
            self.out_block_cache = [None] * self.curr_block_num
            self.lse_block_cache = [None] * self.curr_block_num
        elif new_isp_stride == 0:
            self.curr_isp_stride = 0
            self.curr_block_num = 1
            self.out_block_cache = [None]
            self.lse_block_cache = [None]
        else:
            new_block_num = self.isp_size // new_isp_stride
            assert new_block_num <= self.curr_block_num, "Invalid ISP stride."
            self.curr_isp_stride = new_isp_stride
            if new_block_num != self.curr_block_num:
                self._merge_blocks(new_block_num)
                self.curr_block_num = new_block_num
            self.out_block_cache[next_target_block_id] = None
            self.lse_block_cache[next_target_block_id] = None

    def get_block(self, block_id: int) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
        if block_id >= len(self.out_block_cache):
            logger.error(f"{get_timestep()} | Cache is not ready but trying to get cached value.")
        return self.out_block_cache[block_id], self.lse_block_cache[block_id]

    def store_block(self, block_id: int, out: torch.Tensor, lse: torch.Tensor) -> None:
        """Keep ``(out, lse)`` as block ``block_id``.  A state already in cache form
        (contiguous bf16 or fp16 ``out``, contiguous fp32 ``[B,H,S]`` ``lse`` -- what the
        attention kernel writes for a model that runs in that dtype) is adopted as is; anything
        else goes through one ``dt_cache_store`` pass into fresh cache-form (bf16) tensors."""
        B, S, H, D = out.shape
        in_cache_form = (out.dtype in _hip.HALF_DTYPES and out.is_contiguous() and lse.dtype == torch.float32
                         and tuple(lse.shape) == (B, H, S) and lse.is_contiguous())
        if not in_cache_form:
            slot_out = torch.empty((B, S, H, D), dtype=torch.bfloat16, device=out.device)
            slot_lse = torch.empty((B, H, S), dtype=torch.float32, device=out.device)
            _hip.cache_store(out.contiguous(), lse, slot_out, slot_lse)
            out, lse = slot_out, slot_lse
        self.out_block_cache[block_id] = out
        self.lse_block_cache[block_id] = lse

    def load_block(self, block_id: int, dtype: torch.dtype = torch.float32):
        """Materialise block ``block_id`` as (``out`` in ``dtype``, fp32 ``lse [B,S,H,1]``),
        the form the reference hands to ``update_out_and_lse``; one ``dt_cache_load`` pass."""
        o, l = self.get_block(block_id)
        if l is None:
            return None, None
        return _hip.cache_load(o, l, dtype, dst_lse_bsh=True)

    def clear(self) -> None:
        """cache.py:86-87: logs and keeps every state, as the reference does."""
        logger.warning("============== Clear oCache =================")

    def release(self) -> None:
        """Drop every cached state and the mask-mode arena (no counterpart in the reference, whose
        ``clear`` keeps them): frees the HBM a finished generation holds."""
        self.out_block_cache = [None] * self.curr_block_num
        self.lse_block_cache = [None] * self.curr_block_num
        self.arena_out = self.arena_lse = self.diag_out = self.diag_lse = None
        self.arena_valid = []
        self.arena_refused = None

    # ---- mask-mode arena --------------------------------------------------------------------------
    def ensure_arena(self, n_chunks: int, B: int, Sq: int, H: int, D: int, device,
                     dtype: torch.dtype = torch.bfloat16) -> bool:
        """Make sure the mask-mode arena of this layer exists.  Returns False when it does not fit:
        the arena (``n_chunks + 1`` states) is only allocated if the current allocation plus its size
        stays under ``memory_constraint`` -- the same probe and budget as ``pass_memory_check``
        (cache.py:103-128) -- and a layer without arena recomputes every chunk on every call, which is
        what the reference's guard falls back to (core/attention.py:97-98: stride forced to N)."""
        shape = (n_chunks, B, Sq, H, D)
        if (self.arena_out is not None and tuple(self.arena_out.shape) == shape and self.arena_out.device == device
                and self.arena_out.dtype == dtype):
            return True
        if self.arena_refused == shape:
            return False
        self.arena_out = self.arena_lse = self.diag_out = self.diag_lse = None
        need_mb = (n_chunks + 1) * B * Sq * H * (2 * D + 4) / (1024 ** 2)
        now = self.memory_probe()
        if now + need_mb > self.memory_constraint:
            logger.warning(f"T{get_timestep()}L{self.layer_id} | Memory check failed: {now + need_mb:.0f} > "
                           f"{self.memory_constraint:.0f} MB, this layer keeps no state arena and recomputes every chunk")
            self.arena_refused = shape
            self.arena_valid = []
            return False
        self.arena_out = torch.empty(shape, dtype=dtype, device=device)   # bf16, or fp16 for a model run in fp16
        self.arena_lse = torch.empty((n_chunks, B, H, Sq), dtype=torch.float32, device=device)
        self.diag_out = torch.empty((B, Sq, H, D), dtype=dtype, device=device)
        self.diag_lse = torch.empty((B, H, Sq), dtype=torch.float32, device=device)
        self.arena_valid = [False] * n_chunks
        return True

    def report_cache_status(self, layer_id: int) -> None:
        """cache.py:131-207, condensed."""
        filled = sum(o is not None for o in self.out_block_cache)
        marks = " ".join("O" if o is not None else "X" for o in self.out_block_cache)
        logger.info(f"===== Cache Status: Layer {layer_id}, Timestep {get_timestep()} =====")
        logger.info(f"ISP size {self.isp_size} stride {self.curr_isp_stride} blocks {filled}/{self.curr_block_num} [{marks}]")
        if self.block_size_mb:
            logger.info(f"block {self.block_size_mb:.2f} MB, cache {self.block_size_mb * filled:.2f} MB")
