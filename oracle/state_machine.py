"""``proCache`` and ``proAttention.attn`` restated (CPU oracle; test infrastructure only).

The reference runs one process per ring rank and moves K/V chunks between them
with batched isend/irecv (``core/attention.py:37-71``,
``core/group_coordinate.py:643-668``).  This restatement simulates ALL ranks of
the ring in lock step on chunk *ids*: each rank knows which chunk id it holds,
and an exchange replaces it by the id held by the rank it receives from.  Every
exchange is checked for pairing (the rank I receive from must be sending to me),
which is what a real ``batch_isend_irecv`` requires in order not to hang.

Attention states are opaque payloads combined through two callables, so the
same code runs symbolically (payload = tuple of chunk ids, to pin the schedule)
and numerically (payload = ``(out, lse)`` tensors, to pin the arithmetic):

* ``attn_fn(rank, chunk_id) -> payload``      the ``flash_attn_func`` call
* ``merge_fn(a_or_None, b) -> payload``       ``update_out_and_lse``
* ``store_fn(payload) -> payload``            applied when a state enters the
  cache (identity in the reference, which caches fp32; bf16 rounding when
  mirroring an HBM cache that stores bf16).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, List, Optional, Sequence, Tuple

Payload = Any


def symbolic_attn(rank: int, chunk_id: int) -> Tuple[int, ...]:
    return (chunk_id,)


def symbolic_merge(a: Optional[Tuple[int, ...]], b: Tuple[int, ...]) -> Tuple[int, ...]:
    return tuple(b) if a is None else tuple(a) + tuple(b)


class CacheOracle:
    """core/cache.py:9-128 (bookkeeping only; payloads are opaque)."""

    def __init__(self, isp_size: int, merge_fn: Callable = symbolic_merge,
                 memory_ok: Optional[Callable[["CacheOracle", int], bool]] = None,
                 memory_probe: Optional[Callable[[], float]] = None, block_size_mb: Optional[float] = None,
                 memory_constraint: float = float("inf")):
        self.isp_size = isp_size  # cache.py:12
        self.curr_isp_stride = isp_size  # cache.py:13
        self.curr_block_num = isp_size  # cache.py:14
        self.slots: List[Optional[Payload]] = [None] * isp_size  # cache.py:17-18
        self.merge_fn = merge_fn
        self.memory_ok = memory_ok
        # the guard's three quantities in MB (cache.py:21-22, :89-101, :121): the device-memory
        # reading is a callable so that a test can make the guard trip at a chosen call
        self.memory_probe = memory_probe
        self.block_size_mb = block_size_mb
        self.memory_constraint = memory_constraint

    def _merge_blocks(self, new_block_num: int) -> None:
        # cache.py:28-46
        assert self.curr_block_num % new_block_num == 0, f"Invalid block number {new_block_num} for merging."
        group = self.curr_block_num // new_block_num
        new_slots: List[Optional[Payload]] = [None] * new_block_num
        for i in range(new_block_num):
            merged = None
            for j in range(group):
                st = self.slots[i * group + j]
                if st is not None:  # cache.py:39
                    merged = self.merge_fn(merged, st)  # cache.py:42
            new_slots[i] = merged
        self.slots = new_slots

    def update_cache_blocks(self, new_isp_stride: int, next_target_block_id: int) -> None:
        # cache.py:49-72
        if new_isp_stride == self.isp_size:
            self.curr_isp_stride = self.isp_size
            self.curr_block_num = self.isp_size
            self.slots = [None] * self.curr_block_num
        elif new_isp_stride == 0:
            self.curr_isp_stride = 0
            self.curr_block_num = 1
            self.slots = [None]
        else:
            new_block_num = self.isp_size // new_isp_stride
            assert new_block_num <= self.curr_block_num, "Invalid ISP stride."  # cache.py:65
            self.curr_isp_stride = new_isp_stride
            if new_block_num != self.curr_block_num:
                self._merge_blocks(new_block_num)
                self.curr_block_num = new_block_num
            self.slots[next_target_block_id] = None  # cache.py:71-72

    def get_block(self, block_id: int) -> Optional[Payload]:
        # cache.py:75-80: an id past the end raises IndexError after logging
        return self.slots[block_id]

    def store_block(self, block_id: int, state: Payload) -> None:
        # cache.py:82-84
        self.slots[block_id] = state

    def pass_memory_check(self, next_isp_stride: int) -> bool:
        # cache.py:103-128 with the device-memory reading made injectable
        if next_isp_stride == self.isp_size:  # cache.py:104-105
            return True
        if self.memory_ok is not None:  # a test's own verdict
            return bool(self.memory_ok(self, next_isp_stride))
        if self.memory_probe is None or self.block_size_mb is None:  # cache.py:115-116
            return True
        active = sum(s is not None for s in self.slots)  # cache.py:106-109
        predicted = self.isp_size // next_isp_stride  # cache.py:117
        if predicted <= active:  # cache.py:118-119
            return True
        add = self.block_size_mb * (predicted - active)  # cache.py:121
        return not (self.memory_probe() + add > self.memory_constraint)  # cache.py:122-127


@dataclass
class CallTrace:
    """Everything one rank did in one ``attn`` call (the schedule to match bit-exactly)."""
    timestep: int
    layer_id: int
    rank: int
    curr_stride: int
    next_stride: int
    reuse_probed: List[int] = field(default_factory=list)      # block ids looked up (attention.py:110-112)
    reuse_merged: List[int] = field(default_factory=list)      # those that were non-empty (attention.py:115-116)
    computed: List[Tuple[int, str]] = field(default_factory=list)  # (chunk id, 'local'|'own'|'fresh') in launch order
    stores: List[Tuple[int, Tuple[int, ...]]] = field(default_factory=list)  # (slot id, chunk ids of the fresh state)
    flushes: List[Tuple[int, ...]] = field(default_factory=list)  # chunk ids of each fresh state merged into out
    target_after: int = 0
    nblk_after: int = 0
    occupancy_after: List[bool] = field(default_factory=list)
    out: Payload = None


class RingOracle:
    """All ``N`` ranks of ``proAttention`` for ONE layer, stepped in lock step.

    ``curr_stride_fn(t) / next_stride_fn(t)`` give the strides for this layer
    (``RedundancyMap.get_curr_isp_stride / get_next_isp_stride``).
    """

    def __init__(self, isp_size: int, layer_id: int = 0, use_ditango: bool = True,
                 attn_fn: Callable = symbolic_attn, merge_fn: Callable = symbolic_merge,
                 store_fn: Callable = lambda s: s,
                 memory_ok: Optional[Callable] = None, small_ring_stride: int = 8,
                 memory_probe: Optional[Callable[[], float]] = None, block_size_mb: Optional[float] = None,
                 memory_constraint: float = float("inf")):
        N = isp_size
        self.N = N
        self.layer_id = layer_id
        self.use_ditango = use_ditango  # attention.py:30
        self.small_ring_stride = small_ring_stride  # attention.py:31
        self.attn_fn = attn_fn
        self.merge_fn = merge_fn
        self.store_fn = store_fn
        # attention.py:27: local_chunk_id // isp_size == 0 for every rank
        self.target = [r // N for r in range(N)]
        self.caches = [CacheOracle(N, merge_fn, memory_ok, memory_probe, block_size_mb, memory_constraint)
                       for _ in range(N)]  # attention.py:28

    # -- one synchronous exchange over all ranks -------------------------------------------
    def _exchange(self, held: List[int], posts: List[Optional[Tuple[int, int]]]) -> List[int]:
        """posts[r] = (dst, src) or None.  Returns the chunk ids received."""
        N = self.N
        active = [r for r in range(N) if posts[r] is not None]
        assert len(active) in (0, N), "some ranks post a ring exchange while others do not -> the real ring hangs"
        new = list(held)
        for r in active:
            dst, src = posts[r]
            assert posts[src][0] == r, f"rank {r} receives from {src}, but {src} sends to {posts[src][0]}"
            assert posts[dst][1] == r, f"rank {r} sends to {dst}, but {dst} receives from {posts[dst][1]}"
            new[r] = held[src]
        return new

    def call(self, timestep: int, curr_stride: int, next_stride: int) -> List[CallTrace]:
        """attention.py:74-237 for all ranks."""
        N = self.N
        curr = curr_stride
        traces = [CallTrace(timestep, self.layer_id, r, curr, next_stride) for r in range(N)]
        nxt = [next_stride] * N
        for r in range(N):
            if not self.caches[r].pass_memory_check(nxt[r]):  # attention.py:97-98
                nxt[r] = N
            traces[r].next_stride = nxt[r]
        assert N % curr == 0, f"Does not support this ISP stride {curr} for SP size {N}"  # attention.py:100
        nblk = N // curr  # attention.py:102
        out: List[Payload] = [None] * N
        tb = [0] * N
        lb = [0] * N
        for r in range(N):
            lb[r] = r // curr  # attention.py:103
            tb[r] = self.target[r] // curr  # attention.py:104
            # 1. reuse cached blocks (attention.py:107-116)
            if curr == N:
                self.target[r] = r
            else:
                for i in range(nblk - 1):
                    b = (tb[r] + 1 + i) % nblk
                    traces[r].reuse_probed.append(b)
                    st = self.caches[r].get_block(b)
                    if st is not None:
                        traces[r].reuse_merged.append(b)
                        out[r] = self.merge_fn(out[r], st)
        # 2. first KV fetch (attention.py:120-145)
        held = list(range(N))
        posts: List[Optional[Tuple[int, int]]] = [None] * N
        for r in range(N):
            if self.target[r] != r:
                stride_blocks = (tb[r] - lb[r]) % nblk  # attention.py:123
                send_block = (lb[r] - stride_blocks) % nblk  # attention.py:124
                inner = r % curr  # attention.py:125
                recv_rank = tb[r] * curr + inner  # attention.py:127
                send_rank = send_block * curr + inner  # attention.py:128
                posts[r] = (send_rank, recv_rank)
        fetched = self._exchange(held, posts)
        for r in range(N):
            if posts[r] is not None:
                st = self.attn_fn(r, held[r])  # local chunk, attention.py:137-143
                traces[r].computed.append((held[r], "local"))
                out[r] = self.merge_fn(out[r], st)  # attention.py:144
        held = fetched  # attention.py:145

        # 3. target block (attention.py:148-201)
        upd = 1 if curr == N else curr  # attention.py:148
        nlarge = 1
        ss = curr
        if curr > self.small_ring_stride and self.use_ditango:  # attention.py:152
            assert curr % self.small_ring_stride == 0
            nlarge = curr // self.small_ring_stride
            ss = self.small_ring_stride
        fresh: List[Payload] = [None] * N
        fresh_ids: List[Tuple[int, ...]] = [()] * N
        cnt = [0] * N
        for i in range(nlarge):
            for j in range(ss):
                posts = [None] * N
                for r in range(N):
                    small_off = r // ss * ss  # attention.py:157
                    large_off = r // curr * curr  # attention.py:158
                    if j + 1 != ss:  # attention.py:169-174
                        posts[r] = ((r - 1) % ss + small_off, (r + 1) % ss + small_off)
                    elif i + 1 != nlarge:  # attention.py:177-183
                        posts[r] = ((r - ss) % curr + large_off, (r + ss) % curr + large_off)
                nxt_held = self._exchange(held, posts)
                for r in range(N):
                    st = self.attn_fn(r, held[r])  # attention.py:185-191
                    if lb[r] == tb[r] and i == 0 and j == 0:  # attention.py:193-194
                        traces[r].computed.append((held[r], "own"))
                        out[r] = self.merge_fn(out[r], st)
                    else:  # attention.py:196
                        traces[r].computed.append((held[r], "fresh"))
                        fresh[r] = self.merge_fn(fresh[r], st)
                        fresh_ids[r] = fresh_ids[r] + (held[r],)
                    cnt[r] += 1
                held = nxt_held  # attention.py:200-201
                for r in range(N):
                    if cnt[r] == upd:  # attention.py:204
                        if fresh[r] is not None:
                            if nxt[r] != N:  # attention.py:207
                                slot = self.target[r] if curr == N else tb[r]  # attention.py:208-211
                                stored = self.store_fn(fresh[r])
                                self.caches[r].store_block(slot, stored)
                                traces[r].stores.append((slot, fresh_ids[r]))
                                # the reference merges the very tensor it cached (attention.py:213)
                                fresh[r] = stored
                            traces[r].flushes.append(fresh_ids[r])
                            out[r] = self.merge_fn(out[r], fresh[r])  # attention.py:213
                        self.target[r] = (self.target[r] + cnt[r]) % N  # attention.py:214
                        fresh[r] = None
                        fresh_ids[r] = ()
                        cnt[r] = 0
        # 5. cache management (attention.py:219-220)
        for r in range(N):
            self.caches[r].update_cache_blocks(nxt[r], self.target[r] // nxt[r])
            traces[r].target_after = self.target[r]
            traces[r].nblk_after = self.caches[r].curr_block_num
            traces[r].occupancy_after = [s is not None for s in self.caches[r].slots]
            traces[r].out = out[r]
        return traces


def strides_from_dividers(N: int, dividers: Sequence[int]) -> Tuple[List[int], List[int]]:
    """Per-step (curr, next) strides of one layer from its divider column.

    core/redundancy_map.py:49-87 with ``base_weight = N``: ``N // divider``
    (1 when ``N < divider``), and ``N`` after the last step.
    """
    T = len(dividers)

    def stride(d: int) -> int:
        if N < d:
            return 1
        assert N % d == 0, f"Invalid divider {d} for base weight {N}"
        return max(N // d, 1)

    curr = [stride(int(d)) for d in dividers]
    nxt = [curr[t + 1] if t + 1 < T else N for t in range(T)]
    return curr, nxt


def legal_divider_column(dividers: Sequence[int]) -> bool:
    """The transition rule ``_refine_divider_map`` enforces between consecutive
    steps (core/redundancy_map.py:306-319): previous == 1, or current <= previous.
    Equivalent to the cache's ``new_block_num <= curr_block_num`` (cache.py:65)."""
    for t in range(1, len(dividers)):
        if dividers[t - 1] != 1 and dividers[t] > dividers[t - 1]:
            return False
    return True
