"""Cached block attention: the per-layer driver.

API of the reference's ``proAttention`` (core/attention.py:20-419):
``proAttention(layer_id, isp_group).attn(query, key, value)`` with inputs
``[B, S, H, D]`` bf16 (or fp16) and an fp32 result of the same shape.

One GPU plays one sequence-parallel rank.  Where the reference interleaves ring
hops, one ``flash_attn_func`` call per chunk and one eager merge chain per state,
this driver first derives the whole call's schedule on the host from the same
integer state (stride table, rotating target pointer, cache occupancy), then
issues

1. ONE attention launch that produces every state of the call (``dt_attn_jobs_fwd``:
   the local chunk, and the fresh state of the target block as a single multi-chunk
   job written straight into its cache tensors), and
2. ONE fused N-way merge (``dt_merge_states``) over the cached states, the local
   state and the fresh states.

Which chunk the ring would have delivered at each hop follows from tracking, as
integers, the chunk id every ring position holds (``plan_call``); the chunk order, the reuse set, the cache writes and the pointer
movement match the reference step for step, including the case in which it
merges the local chunk twice (core/attention.py:120-145 followed by :193-194).

Mask mode (an addition, see ``RedundancyMap.set_chunk_mask``): the chunks to
compute come from a device-resident schedule and every state lives in a
contiguous per-layer arena.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Tuple

import torch

from .. import _hip
from ..logger import init_logger
from ..timer import get_timer
from ..utils import get_timestep
from .cache import proCache
from .config import get_config
from .redundancy_map import get_redundancy_map

logger = init_logger(__name__)


@dataclass
class Job:
    chunks: Tuple[int, ...]   # KV chunk ids attended to as one concatenated sequence
    kind: str                 # 'local' (computed while the first fetch is in flight), 'own', 'fresh'
    store_slot: Optional[int] = None  # cache block the state is stored in, if any


@dataclass
class CallPlan:
    """The schedule of one ``attn`` call (what has to match the reference bit for bit)."""
    timestep: int
    layer_id: int
    rank: int
    curr_stride: int
    next_stride: int
    reuse_probed: List[int] = field(default_factory=list)
    reuse_merged: List[int] = field(default_factory=list)
    computed: List[Tuple[int, str]] = field(default_factory=list)
    jobs: List[Job] = field(default_factory=list)
    stores: List[Tuple[int, Tuple[int, ...]]] = field(default_factory=list)
    flushes: List[Tuple[int, ...]] = field(default_factory=list)
    target_after: int = 0
    nblk_after: int = 0
    occupancy_after: List[bool] = field(default_factory=list)


def plan_call(N: int, r: int, curr: int, nxt: int, targets: List[int], use_ditango: bool = True,
              small_ring_stride: int = 8) -> Tuple[CallPlan, List[int]]:
    """Schedule of one call from the integer state alone (core/attention.py:100-216).

    ``targets[x]`` is the rotating target pointer of ring position ``x``; all positions
    are tracked because which chunk a hop delivers depends on what the NEIGHBOUR fetched:
    after a stride-1 step the pointers of one block's ranks can point into different
    target blocks, and the reference then hands chunks of other blocks round the ring.
    ``held[x]`` is the chunk id position ``x`` has in hand; an exchange replaces it by
    the id held by the position it receives from (ring sends to ``x-1``, receives from
    ``x+1`` inside a small ring of ``ss`` positions, :160-161; an inter-ring hop receives
    from ``x+ss`` inside the block, :162-163).

    Returns (plan of position ``r`` without the cache-dependent fields, new pointers).
    """
    assert N % curr == 0, f"Does not support this ISP stride {curr} for SP size {N}"
    plan = CallPlan(0, 0, r, curr, nxt)
    nblk = N // curr
    targets = list(targets)
    tb_of = [targets[x] // curr for x in range(N)]  # read before the pointer reset (:104)
    lb, tb = r // curr, tb_of[r]
    if curr == N:
        targets = list(range(N))  # :107-108
    else:
        plan.reuse_probed = [(tb + 1 + i) % nblk for i in range(nblk - 1)]
    # first fetch (:120-145): position x takes the chunk of the same inner offset in its target block
    held = list(range(N))
    fetching = [targets[x] != x for x in range(N)]
    if any(fetching):
        if not all(fetching):
            raise RuntimeError("ring positions disagree on whether to fetch first: the reference's exchange would hang "
                               "(the first step of a run has to be a full-stride step)")
        src = [tb_of[x] * curr + x % curr for x in range(N)]
        dst = [((x // curr - (tb_of[x] - x // curr)) % nblk) * curr + x % curr for x in range(N)]
        for x in range(N):
            if dst[src[x]] != x:
                raise RuntimeError(f"unpaired first fetch at ring position {x}: the reference's exchange would hang")
        held = [held[src[x]] for x in range(N)]
        plan.computed.append((r, "local"))
        plan.jobs.append(Job((r,), "local"))
    upd = 1 if curr == N else curr
    ss = curr
    if curr > small_ring_stride and use_ditango:
        assert curr % small_ring_stride == 0, f"Does not support this ISP stride {curr} for overlap ring strategy"
        ss = small_ring_stride
    nlarge = curr // ss
    fresh: List[int] = []
    cnt = 0
    for i in range(nlarge):
        for j in range(ss):
            c = held[r]
            if lb == tb and i == 0 and j == 0:
                plan.computed.append((c, "own"))
                plan.jobs.append(Job((c,), "own"))
            else:
                plan.computed.append((c, "fresh"))
                fresh.append(c)
            cnt += 1
            if j + 1 != ss:
                held = [held[(x + 1) % ss + x // ss * ss] for x in range(N)]
            elif i + 1 != nlarge:
                held = [held[(x + ss) % curr + x // curr * curr] for x in range(N)]
            if cnt == upd:
                if fresh:
                    slot = None
                    if nxt != N:
                        slot = targets[r] if curr == N else tb
                        plan.stores.append((slot, tuple(fresh)))
                    plan.flushes.append(tuple(fresh))
                    plan.jobs.append(Job(tuple(fresh), "fresh", slot))
                targets = [(tg + cnt) % N for tg in targets]  # every position flushes in the same iteration
                fresh = []
                cnt = 0
    plan.target_after = targets[r]
    return plan, targets


_warned_cast = set()


def _kernel_input(t: torch.Tensor) -> torch.Tensor:
    """The kernels run in bf16 or fp16, the two dtypes flash_attn_func takes: such inputs pass as they are
    (fp16 on the fp16 MFMA, states and cache slots in fp16).  fp32 inputs (the reference's CPU-runnable case
    is stated in fp32) are rounded to bf16 here, once, explicitly: the result is then the attention of the
    ROUNDED inputs, which differs from fp32 attention of the unrounded ones by the input rounding
    (2^-9 relative per element)."""
    if t is None or t.dtype in _hip.HALF_DTYPES:
        return t
    if t.dtype != torch.float32:
        raise TypeError(f"attention inputs must be bf16, fp16 or fp32, got {t.dtype}")
    if t.dtype not in _warned_cast:
        _warned_cast.add(t.dtype)
        logger.warning(f"attention inputs of dtype {t.dtype} are rounded to bf16 at the kernel boundary")
    return t.to(torch.bfloat16)


def _as4d(t: torch.Tensor, B: int) -> torch.Tensor:
    """Packed ``[B*S, H, D]`` (the varlen entry's layout) viewed as ``[B, S, H, D]``, in the kernels' dtype."""
    t = _kernel_input(t)
    return t if t.dim() == 4 else t.view(B, t.shape[0] // B, t.shape[1], t.shape[2])


class proAttention:
    def __init__(self, layer_id: int, isp_group, dry_run: bool = False):
        self.group = isp_group
        self.isp_size = self.group.world_size
        self.global_rank = getattr(get_config(), "rank", 0) if get_config() is not None else 0
        self.local_chunk_id = self.group.rank_in_group
        self.layer_id = layer_id
        self.target_chunk_id = self.local_chunk_id // self.isp_size  # core/attention.py:27
        # pointers of all ring positions (each starts at position // isp_size = 0); see plan_call
        self._ring_targets = [x // self.isp_size for x in range(self.isp_size)]
        self.cache = proCache(isp_size=self.isp_size, layer_id=layer_id)
        cfg = get_config()
        self.use_ditango = cfg.use_ditango if cfg is not None else True
        self.small_ring_stride = 8
        self.measure_memory = False
        self.dry_run = dry_run  # plan and book-keep only (host tests of the schedule); computes nothing
        self.last_plan: Optional[CallPlan] = None
        self.last_lse: Optional[torch.Tensor] = None  # merged lse of the last call, fp32 [B,S,H,1]
        # dtype of the returned tensor.  The reference returns fp32 and every caller casts right away
        # (attention_processor.py:80, step/attentions.py:98); torch.bfloat16 here lets the merge kernel
        # write the bf16 the out-projection consumes: half the result bytes and no separate cast pass.
        self.out_dtype = torch.float32
        # True: the caller folded softmax_scale * log2(e) into the query before rounding it to bf16
        # (ditango_amd.producer.prepare_qk(..., fold_softmax_scale=...), or the QK-norm weight): the
        # kernels then skip the scaling (a quarter of the softmax's vector instructions).  Not what the
        # reference's callers pass (flash_attn_func scales inside, core/attention.py:137-143).
        self.q_prescaled = False
        # What happens to fp32 inputs (flash_attn_func takes none; the reference's CPU-runnable configuration is
        # stated in fp32): "round" = rounded to bf16 at the kernel boundary, the bf16 MFMA kernels run;
        # "exact" = every fresh state is computed in fp32 from the fp32 tensors (dt_attn_chunk_f32_fwd, a
        # plain vector-ALU kernel for small problems) and only cached states are rounded to bf16.
        self.fp32_inputs = "round"
        self._exact_f32 = False
        # while a variable-length call runs: (cu_seqlens_q, chunk -> cu_seqlens_kv) as host lists, or a
        # _DeviceSegmentSource when the boundaries are device tensors that the host never reads
        self._segments = None
        if self.layer_id == 0:
            logger.info(f"R{self.global_rank}L{layer_id} | cached block attention on HIP kernels (gfx950)")

    _MAX_JOB_CHUNKS = 32  # chunks of one block computed as one job (a launch addresses _hip.DT_MAX_CHUNKS)

    # ---- stride mode ------------------------------------------------------------------------------
    def _strides(self, timestep: int) -> Tuple[int, int]:
        rm = get_redundancy_map()
        return rm.get_curr_isp_stride(timestep, self.layer_id), rm.get_next_isp_stride(timestep, self.layer_id)

    @get_timer("oAttn")
    def attn(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor) -> Optional[torch.Tensor]:
        """query ``[B,Sq,H,D]``, key/value ``[B,Sk,H,D]`` = this rank's shard (bf16 or fp16).
        Returns fp32 ``[B,Sq,H,D]`` (core/attention.py:74-237)."""
        rm = get_redundancy_map()
        self._exact_f32 = (not self.dry_run and self.fp32_inputs == "exact" and query is not None
                           and query.dtype == torch.float32)
        if not self.dry_run and not self._exact_f32:
            query, key, value = _kernel_input(query), _kernel_input(key), _kernel_input(value)
        if rm is not None and rm.chunk_mask is not None and not self.dry_run:
            return self._attn_masked_f32(query, key, value) if self._exact_f32 else self._attn_masked(query, key, value)
        timestep = get_timestep()
        N, r = self.isp_size, self.local_chunk_id
        curr, nxt = self._strides(timestep)
        if timestep == 0 and value is not None:
            self.cache.set_block_size_mb(value)  # :93-94
        # :97-98: an over-budget prediction turns the announced stride into N for this call only -- the next
        # call reads its stride from the map again and probes a cache that was reset to N empty slots
        if not self.cache.pass_memory_check(nxt, self.layer_id):
            nxt = N
        if self._ring_targets[r] != self.target_chunk_id:  # the pointer was set from outside: same offset everywhere
            shift = (self.target_chunk_id - self._ring_targets[r]) % N
            self._ring_targets = [(tg + shift) % N for tg in self._ring_targets]
        plan, new_targets = plan_call(N, r, curr, nxt, self._ring_targets, self.use_ditango, self.small_ring_stride)
        new_target = new_targets[r]
        plan.timestep, plan.layer_id = timestep, self.layer_id

        # 1. cached states of the blocks that are not recomputed (:107-116)
        merge_outs, merge_lses = [], []
        for b in plan.reuse_probed:
            c_out, c_lse = self.cache.get_block(b)
            if c_lse is not None:
                plan.reuse_merged.append(b)
                merge_outs.append(c_out)
                merge_lses.append(c_lse)

        out = None
        if self.dry_run:
            for job in plan.jobs:
                if job.store_slot is not None:
                    self.cache.out_block_cache[job.store_slot] = job.chunks
                    self.cache.lse_block_cache[job.store_slot] = job.chunks
        else:
            out = self._execute(plan, query, key, value, merge_outs, merge_lses, self._segments)

        # 4./5. pointer and cache management (:214, :219-220)
        self.target_chunk_id = new_target
        self._ring_targets = new_targets
        if self.dry_run:
            self._dry_update_cache(nxt, new_target // nxt)
        else:
            self.cache.update_cache_blocks(nxt, new_target // nxt)
        plan.nblk_after = self.cache.curr_block_num
        plan.occupancy_after = [o is not None for o in self.cache.out_block_cache]
        self.last_plan = plan
        if out is not None:
            rm.record_out_redundancy(timestep=timestep, layer_id=self.layer_id, curr_out=out)  # :233-236
        return out

    def _dry_update_cache(self, nxt: int, next_target_block: int) -> None:
        """``update_cache_blocks`` on occupancy tokens (tuples of chunk ids) instead of tensors."""
        cache = self.cache
        if nxt != self.isp_size and nxt != 0:
            new_n = self.isp_size // nxt
            assert new_n <= cache.curr_block_num, "Invalid ISP stride."
            if new_n != cache.curr_block_num:
                group = cache.curr_block_num // new_n
                merged = []
                for i in range(new_n):
                    parts = [cache.out_block_cache[i * group + j] for j in range(group)
                             if cache.out_block_cache[i * group + j] is not None]
                    merged.append(tuple(c for p in parts for c in p) if parts else None)
                cache.out_block_cache = merged
                cache.lse_block_cache = list(merged)
                cache.curr_block_num = new_n
            cache.curr_isp_stride = nxt
            cache.out_block_cache[next_target_block] = None
            cache.lse_block_cache[next_target_block] = None
        else:
            cache.update_cache_blocks(nxt, next_target_block)

    def _chunk_f32(self, c: int, key, value, B: int):
        """fp32 K/V of chunk ``c`` as ``[B,S,H,D]`` (exact-fp32 mode: no rounding)."""
        k_c, v_c = (key, value) if (c == self.local_chunk_id and key is not None) else self.group.kv_chunk(c)
        if k_c.dtype != torch.float32 or v_c.dtype != torch.float32:
            raise TypeError("fp32_inputs = 'exact' needs fp32 K/V chunks as well")
        k_c = k_c if k_c.dim() == 4 else k_c.view(B, k_c.shape[0] // B, k_c.shape[1], k_c.shape[2])
        v_c = v_c if v_c.dim() == 4 else v_c.view(B, v_c.shape[0] // B, v_c.shape[1], v_c.shape[2])
        return k_c, v_c

    def _job_state_f32(self, query, chunks, key, value):
        """The fp32 state of ``query`` against the concatenation of ``chunks``, computed in fp32."""
        if self._segments is not None:
            raise NotImplementedError("fp32_inputs = 'exact' does not cover variable-length calls")
        B = query.shape[0]
        states = [_hip.attn_chunk_f32_fwd(query, *self._chunk_f32(c, key, value, B)) for c in chunks]
        if len(states) == 1:
            return states[0]
        return _hip.merge_states([s[0] for s in states], [s[1] for s in states], dst_dtype=torch.float32)

    def _execute(self, plan: CallPlan, query, key, value, merge_outs, merge_lses, segments=None) -> torch.Tensor:
        B, Sq, H, D = query.shape
        N, r = self.isp_size, self.local_chunk_id
        dev = query.device
        if self._exact_f32:
            seen = {}
            for job in plan.jobs:
                if job.chunks not in seen:
                    seen[job.chunks] = self._job_state_f32(query, job.chunks, key, value)
                o, l = seen[job.chunks]
                if job.store_slot is not None:
                    self.cache.store_block(job.store_slot, o, l)      # rounded to bf16 on its way into the cache
                merge_outs.append(o)
                merge_lses.append(l)
            out, lse = _hip.merge_states(merge_outs, merge_lses, dst_dtype=self.out_dtype, dst_lse_bsh=True)
            self.last_lse = lse
            return out
        # chunk table: the local chunk is (key, value); the others come from the ring stand-in
        needed = sorted({c for job in plan.jobs for c in job.chunks})
        ks: List[torch.Tensor] = []
        vs: List[torch.Tensor] = []
        index = {}
        for c in needed:
            index[c] = len(ks)
            k_c, v_c = (key, value) if c == r else self.group.kv_chunk(c)
            ks.append(_as4d(k_c, B))
            vs.append(_as4d(v_c, B))
        # one launch for all distinct states; a chunk computed twice by the reference
        # (local + own) is computed once and merged twice
        job_lists, dests, seen = [], [], {}
        pieced = []  # states computed in pieces: [(o, l) of the first piece = destination, the others...]
        dev_seg = segments if isinstance(segments, _DeviceSegmentSource) else None
        q_ranges, kv_ranges = ([], []) if segments is not None and dev_seg is None else (None, None)
        job_segs = [] if dev_seg is not None else None
        states = []
        for job in plan.jobs:
            if job.chunks in seen and job.store_slot is None:
                states.append(seen[job.chunks])
                continue
            o = torch.empty((B, Sq, H, D), dtype=query.dtype, device=dev)
            l = torch.empty((B, H, Sq), dtype=torch.float32, device=dev)
            if len(set(job.chunks)) > self._MAX_JOB_CHUNKS:
                # a block of more chunks than one launch addresses (rings of 128 positions and more): its
                # state is computed in pieces that are folded into (o, l) behind the attention launch
                pieces = [job.chunks[i:i + self._MAX_JOB_CHUNKS] for i in range(0, len(job.chunks), self._MAX_JOB_CHUNKS)]
                piece_states = [(o, l)] + [(torch.empty_like(o), torch.empty_like(l)) for _ in pieces[1:]]
                pieced.append(piece_states)
            else:
                pieces, piece_states = [job.chunks], [(o, l)]
            if segments is None:
                for piece, st in zip(pieces, piece_states):
                    job_lists.append([index[c] for c in piece])
                    dests.append(st)
            elif len(pieces) > 1:
                raise NotImplementedError("variable-length calls with blocks of more than "
                                          f"{self._MAX_JOB_CHUNKS} chunks are not supported")
            elif dev_seg is not None:
                # one kernel job per segment; the kernel reads the segment's rows and keys from device memory
                for i in range(dev_seg.n_seg):
                    job_lists.append([index[c] for c in job.chunks])
                    dests.append((o, l))
                    job_segs.append(i)
            else:
                # one kernel job per segment: its query rows against its key rows of every chunk
                cu_q, cu_kv_of = segments
                for i in range(len(cu_q) - 1):
                    job_lists.append([index[c] for c in job.chunks])
                    dests.append((o, l))
                    q_ranges.append((cu_q[i], cu_q[i + 1] - cu_q[i]))
                    kv_ranges.append([(cu_kv_of(c)[i], cu_kv_of(c)[i + 1] - cu_kv_of(c)[i]) for c in job.chunks])
            seen[job.chunks] = (o, l)
            states.append((o, l))
        if job_lists:
            table = _hip.ChunkTable(ks, vs)
            if dev_seg is not None:
                _hip.attn_jobs_fwd(query, table, job_lists, [d[0] for d in dests], [d[1] for d in dests],
                                   q_prescaled=self.q_prescaled, dev_segments=dev_seg.over(needed), job_segments=job_segs)
            else:
                _hip.attn_jobs_fwd(query, table, job_lists, [d[0] for d in dests], [d[1] for d in dests],
                                   q_ranges=q_ranges, kv_ranges=kv_ranges, workspace=_hip.attn_workspace(dev),
                                   q_prescaled=self.q_prescaled)
        for piece_states in pieced:
            _hip.merge_states([s[0] for s in piece_states], [s[1] for s in piece_states],
                              dst_out=piece_states[0][0], dst_lse=piece_states[0][1])
        for job, (o, l) in zip(plan.jobs, states):
            if job.store_slot is not None:
                self.cache.store_block(job.store_slot, o, l)  # :207-211
            merge_outs.append(o)
            merge_lses.append(l)
        out, lse = _hip.merge_states(merge_outs, merge_lses, dst_dtype=self.out_dtype, dst_lse_bsh=True)
        self.last_lse = lse
        return out

    # ---- mask mode ----------------------------------------------------------------------------------
    def _attn_masked(self, query, key, value) -> torch.Tensor:
        rm = get_redundancy_map()
        t, l = get_timestep(), self.layer_id
        C = rm.chunk_mask.shape[2]
        diag = rm.mask_diag
        B, Sq, H, D = query.shape
        cache = self.cache
        row = rm.chunk_mask[t, l]
        ks, vs = [], []
        for c in range(C):
            use_local = (c == self.local_chunk_id and c == diag and key is not None)
            k_c, v_c = (key, value) if use_local else self.group.kv_chunk(c)
            ks.append(_as4d(k_c, B))
            vs.append(_as4d(v_c, B))
        if not cache.ensure_arena(C, B, Sq, H, D, query.device, query.dtype):
            out = self._attn_uncached(query, ks, vs)
            rm.record_out_redundancy(timestep=t, layer_id=l, curr_out=out)
            return out
        for c in range(C):
            if c != diag and row[c] != 0 and not cache.arena_valid[c]:
                raise RuntimeError(f"T{t}L{l}: mask asks to reuse chunk {c} but no state was ever stored for it")
        seg_q = seg_kv = dev_seg = None
        if isinstance(self._segments, _DeviceSegmentSource):
            dev_seg = self._segments.over(range(C))
        elif self._segments is not None:
            # packed variable-length batch: every scheduled chunk runs once per segment
            cu_q, cu_kv_of = self._segments
            seg_q = [(cu_q[i], cu_q[i + 1] - cu_q[i]) for i in range(len(cu_q) - 1)]
            seg_kv = [[(cu_kv_of(c)[i], cu_kv_of(c)[i + 1] - cu_kv_of(c)[i]) for i in range(len(cu_q) - 1)]
                      for c in range(C)]
        ws = _hip.attn_workspace(query.device)
        if not rm.sched_windows:
            n_comp = int(rm.sched_counts_host[t, l, 0])
            _hip.attn_sched_fwd(query, _hip.ChunkTable(ks, vs), rm.sched_compute_ids[t, l], rm.sched_counts[t, l, 0:1],
                                n_comp, cache.arena_out, cache.arena_lse, diag, cache.diag_out, cache.diag_lse,
                                seg_q=seg_q, seg_kv=seg_kv, workspace=ws, q_prescaled=self.q_prescaled,
                                dev_segments=dev_seg)
        else:
            # more chunks than one launch addresses: one launch per window of chunk ids (ordered on the
            # stream, so they can share the workspace)
            for w0, w1, d_w, comp_w, cnt_w, cnt_host_w in rm.sched_windows:
                n_comp = int(cnt_host_w[t, l, 0])
                if n_comp == 0:
                    continue
                if all(k.shape[1] == 0 for k in ks[w0:w1]):
                    # a window without a single key is not launched (a chunk table needs one): the states its
                    # scheduled chunks would have got -- out = 0, lse = -inf, neutral in the merge -- are written here
                    for c in range(w0, w1):
                        if c == diag:
                            cache.diag_out.zero_()
                            cache.diag_lse.fill_(float("-inf"))
                        elif row[c] == 0:
                            cache.arena_out[c].zero_()
                            cache.arena_lse[c].fill_(float("-inf"))
                    continue
                _hip.attn_sched_fwd(query, _hip.ChunkTable(ks[w0:w1], vs[w0:w1]), comp_w[t, l], cnt_w[t, l, 0:1],
                                    n_comp, cache.arena_out[w0:w1], cache.arena_lse[w0:w1], d_w, cache.diag_out,
                                    cache.diag_lse, seg_q=seg_q, seg_kv=None if seg_kv is None else seg_kv[w0:w1],
                                    workspace=ws, q_prescaled=self.q_prescaled,
                                    dev_segments=None if dev_seg is None else dev_seg.window(w0, w1))
        outs, lses = [], []
        for c in range(C):
            if c == diag:
                outs.append(cache.diag_out)
                lses.append(cache.diag_lse)
            else:
                if row[c] == 0:
                    cache.arena_valid[c] = True
                outs.append(cache.arena_out[c])
                lses.append(cache.arena_lse[c])
        out, lse = _hip.merge_states(outs, lses, dst_dtype=self.out_dtype, dst_lse_bsh=True)
        self.last_lse = lse
        rm.record_out_redundancy(timestep=t, layer_id=l, curr_out=out)
        return out

    def _attn_masked_f32(self, query, key, value) -> torch.Tensor:
        """Mask mode on fp32 tensors in exact mode: fresh states in fp32, cached ones bf16 in the arena."""
        rm = get_redundancy_map()
        t, l = get_timestep(), self.layer_id
        C, diag = rm.chunk_mask.shape[2], rm.mask_diag
        B, Sq, H, D = query.shape
        cache = self.cache
        row = rm.chunk_mask[t, l]
        have_arena = cache.ensure_arena(C, B, Sq, H, D, query.device)
        compute = ([diag] if 0 <= diag < C else []) + [c for c in range(C) if c != diag and (row[c] == 0 or not have_arena)]
        outs, lses = [], []
        for c in range(C):
            if c in compute:
                continue
            if not cache.arena_valid[c]:
                raise RuntimeError(f"T{t}L{l}: mask asks to reuse chunk {c} but no state was ever stored for it")
            outs.append(cache.arena_out[c])
            lses.append(cache.arena_lse[c])
        for c in compute:
            o, s = self._job_state_f32(query, (c,), key if c == diag else None, value if c == diag else None)
            if c != diag and have_arena:
                _hip.cache_store(o, s, cache.arena_out[c], cache.arena_lse[c])
                cache.arena_valid[c] = True
            outs.append(o)
            lses.append(s)
        out, lse = _hip.merge_states(outs, lses, dst_dtype=self.out_dtype, dst_lse_bsh=True)
        self.last_lse = lse
        rm.record_out_redundancy(timestep=t, layer_id=l, curr_out=out)
        return out

    def _attn_uncached(self, query, ks, vs) -> torch.Tensor:
        """A layer whose state arena did not fit: attention over all chunks, nothing kept."""
        B, Sq, H, D = query.shape
        dev = query.device
        ids = [c for c in range(len(ks)) if ks[c].shape[1] > 0]
        if not ids:  # no key anywhere: the empty attention state
            self.last_lse = torch.full((B, Sq, H, 1), float("-inf"), dtype=torch.float32, device=dev)
            return torch.zeros((B, Sq, H, D), dtype=self.out_dtype, device=dev)
        pieces = [ids[i:i + self._MAX_JOB_CHUNKS] for i in range(0, len(ids), self._MAX_JOB_CHUNKS)]
        outs = [torch.empty((B, Sq, H, D), dtype=query.dtype, device=dev) for _ in pieces]
        lses = [torch.empty((B, H, Sq), dtype=torch.float32, device=dev) for _ in pieces]
        q_ranges = kv_ranges = None
        jobs, d_out, d_lse = pieces, outs, lses
        if isinstance(self._segments, _DeviceSegmentSource):
            src = self._segments
            jobs, d_out, d_lse, job_segs = [], [], [], []
            for piece, o, l_ in zip(pieces, outs, lses):
                for i in range(src.n_seg):
                    jobs.append(piece)
                    d_out.append(o)
                    d_lse.append(l_)
                    job_segs.append(i)
            _hip.attn_jobs_fwd(query, _hip.ChunkTable(ks, vs), jobs, d_out, d_lse, q_prescaled=self.q_prescaled,
                               dev_segments=src.over(range(len(ks))), job_segments=job_segs)
            out, lse = _hip.merge_states(outs, lses, dst_dtype=self.out_dtype, dst_lse_bsh=True)
            self.last_lse = lse
            return out
        if self._segments is not None:
            cu_q, cu_kv_of = self._segments
            jobs, d_out, d_lse, q_ranges, kv_ranges = [], [], [], [], []
            for piece, o, l_ in zip(pieces, outs, lses):
                for i in range(len(cu_q) - 1):
                    jobs.append(piece)
                    d_out.append(o)
                    d_lse.append(l_)
                    q_ranges.append((cu_q[i], cu_q[i + 1] - cu_q[i]))
                    kv_ranges.append([(cu_kv_of(c)[i], cu_kv_of(c)[i + 1] - cu_kv_of(c)[i]) for c in piece])
        _hip.attn_jobs_fwd(query, _hip.ChunkTable(ks, vs), jobs, d_out, d_lse, q_ranges=q_ranges, kv_ranges=kv_ranges,
                           workspace=_hip.attn_workspace(dev), q_prescaled=self.q_prescaled)
        out, lse = _hip.merge_states(outs, lses, dst_dtype=self.out_dtype, dst_lse_bsh=True)
        self.last_lse = lse
        return out

    # ---- varlen entry (HunyuanVideo) ---------------------------------------------------------------
    @get_timer("varlen oAttn")
    def varlen_attn(self, query, key, value, cu_seqlens_q=None, cu_seqlens_kv=None, max_seqlen_q=None,
                    max_seqlen_kv=None, batch_size=1):
        """core/attention.py:239-419: the same state machine on a packed batch.

        ``query/key/value`` are ``[total, H, D]``; segment ``i`` of the queries
        (rows ``cu_seqlens_q[i]:cu_seqlens_q[i+1]``) attends to segment ``i`` of every KV chunk,
        whose boundaries ``cu_seqlens_kv`` belong to the chunk (the local chunk's are the argument,
        the others come with the chunks: ``LocalRingGroup.set_kv_chunks(..., cu_seqlens_kv=...)``).
        Returns fp32 ``[total, H, D]``.  Without sequence lengths it is ``attn`` (:252-254).
        Each segment runs as attention jobs on row/key sub-ranges of one launch
        (``dt_attn_seg_jobs_fwd``, or ``dt_attn_sched_seg_fwd`` under a per-chunk reuse mask); schedule,
        cache and merge are those of ``attn``."""
        if cu_seqlens_q is None and cu_seqlens_kv is None and max_seqlen_q is None and max_seqlen_kv is None:
            logger.warning("cu_seqlens_q not provided, using normal attention instead.")
            return self.attn(query, key, value)
        total_q, H, D = query.shape
        r = self.local_chunk_id
        on_device = torch.is_tensor(cu_seqlens_q) and cu_seqlens_q.is_cuda
        if on_device and not self.dry_run:
            # the reference's calling convention: int32 cu_seqlens on the GPU.  They stay there -- the kernels read
            # them (dt_attn_varlen_jobs_fwd / dt_attn_sched_varlen_fwd), the host reads none, nothing synchronises
            self._segments = _DeviceSegmentSource(self, cu_seqlens_q, cu_seqlens_kv, max_seqlen_q, total_q)
            cu_q = None
        else:
            cu_q = [int(x) for x in (cu_seqlens_q.tolist() if hasattr(cu_seqlens_q, "tolist") else cu_seqlens_q)]
            local_cu = [int(x) for x in (cu_seqlens_kv.tolist() if hasattr(cu_seqlens_kv, "tolist") else cu_seqlens_kv)]
            assert cu_q[0] == 0 and cu_q[-1] <= total_q and len(local_cu) == len(cu_q), "malformed cu_seqlens"

            def cu_kv_of(c):
                if c == r:
                    return local_cu
                cu = self.group.kv_cu_seqlens(c)
                # (boundaries that were handed over on the GPU beside host-side cu_seqlens_q: one blocking read)
                return [int(x) for x in cu.tolist()] if torch.is_tensor(cu) else cu

            self._segments = (cu_q, cu_kv_of)
        try:
            out = self.attn(query.view(1, total_q, H, D), key.view(1, key.shape[0], H, D),
                            value.view(1, value.shape[0], H, D))
        finally:
            self._segments = None
        # rows outside every segment: flash_attn_varlen_func leaves zeros
        if cu_q is None:
            _hip.zero_rows_from(out.view(total_q, H * D), cu_seqlens_q[-1:])
        elif cu_q[-1] < total_q:
            out[:, cu_q[-1]:] = 0
        return out.view(total_q, H, D)


class _DeviceSegmentSource:
    """The segment boundaries of one variable-length call while they stay in device memory: hands the
    launches a ``_hip.DeviceSegments`` over the chunks they address."""

    def __init__(self, attn: "proAttention", cu_q, local_cu_kv, max_seqlen_q, total_q: int):
        if not (torch.is_tensor(local_cu_kv) and local_cu_kv.is_cuda):
            raise TypeError("cu_seqlens_q is on the GPU, so cu_seqlens_kv must be as well")
        self.attn = attn
        self.cu_q = cu_q.to(torch.int32).contiguous()            # (no-ops for the int32 vectors the callers pass)
        self.local = local_cu_kv.to(torch.int32).contiguous()
        self.max_seqlen_q = int(max_seqlen_q) if max_seqlen_q else int(total_q)
        self.n_seg = self.cu_q.numel() - 1

    def cu_kv(self, c: int):
        if c == self.attn.local_chunk_id:
            return self.local
        cu = self.attn.group.kv_cu_seqlens(c)
        if not torch.is_tensor(cu):                              # a host list beside device boundaries: one small upload
            cu = torch.tensor(list(cu), dtype=torch.int32, device=self.cu_q.device)
        return cu.to(torch.int32).contiguous()

    def over(self, chunk_ids) -> "_hip.DeviceSegments":
        """Boundaries of the chunks ``chunk_ids`` in that order (the local chunk's are the call's ``cu_seqlens_kv``)."""
        return _hip.DeviceSegments(self.cu_q, [self.cu_kv(c) for c in chunk_ids], self.max_seqlen_q)
