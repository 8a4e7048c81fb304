"""ctypes binding of ``libditango_hip.so`` (the C ABI declared in ``include/ditango_hip.h``).

There is no fallback: if the library has not been built, or an entry point
returns an error code, the call raises.  PyTorch only supplies device memory
(``tensor.data_ptr()``) and the stream (``torch.cuda.current_stream()``).
"""
from __future__ import annotations

import ctypes
import os
from pathlib import Path
from typing import List, Optional, Sequence, Tuple

import torch

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libditango_hip.so"

DT_BF16, DT_FP32, DT_FP16 = 0, 1, 2
DT_LSE_BHS, DT_LSE_BSH = 0, 1
DT_NORM_NONE, DT_NORM_RMS, DT_NORM_LAYER = 0, 1, 2
DT_ROPE_NONE, DT_ROPE_INTERLEAVED, DT_ROPE_HALVES = 0, 1, 2
DT_ROUND_NORM_BF16, DT_ROUND_ROPE_BF16, DT_IO_FP16 = 1, 2, 4
DT_ATTN_Q_PRESCALED, DT_ATTN_FP16 = 1, 2
DT_MAX_CHUNKS = 40
DT_MAX_JOBS = 40
DT_MAX_JOB_ENTRIES = 64
DT_MAX_MERGE = 64
DT_MAX_SEGMENTS = 8
DT_NOALLOC_TAIL_SLOTS = 512

c_i32, c_i64, c_f32, c_vp = ctypes.c_int32, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p
_P = ctypes.POINTER

_SIGNATURES = {
    "dt_version": (ctypes.c_int, []),
    "dt_last_error": (ctypes.c_char_p, []),
    "dt_attn_chunk_fwd": (ctypes.c_int, [c_vp, c_vp, c_vp, c_vp, c_vp, c_i32, c_i32, c_i32, c_i32, c_i32,
                                         c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_f32, c_vp]),
    "dt_attn_chunk_f16_fwd": (ctypes.c_int, [c_vp, c_vp, c_vp, c_vp, c_vp, c_i32, c_i32, c_i32, c_i32, c_i32,
                                             c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_f32, c_vp]),
    "dt_attn_chunk_f32_fwd": (ctypes.c_int, [c_vp, c_vp, c_vp, c_vp, c_vp, c_i32, c_i32, c_i32, c_i32, c_i32,
                                             c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_f32, c_vp]),
    "dt_attn_jobs_fwd": (ctypes.c_int, [c_vp, c_i32, c_i32, c_i32, c_i32, c_i64, c_i64, c_i64,
                                        c_i32, _P(c_vp), _P(c_vp), _P(c_i32), _P(c_i64), c_i64, c_i64,
                                        c_i32, _P(c_i32), _P(c_i32), _P(c_vp), _P(c_vp), c_f32, c_vp]),
    "dt_attn_seg_jobs_fwd": (ctypes.c_int, [c_vp, c_i32, c_i32, c_i32, c_i32, c_i64, c_i64, c_i64,
                                            c_i32, _P(c_vp), _P(c_vp), _P(c_i32), _P(c_i64), c_i64, c_i64,
                                            c_i32, _P(c_i32), _P(c_i32), _P(c_i32), _P(c_i32), _P(c_i32), _P(c_i32),
                                            _P(c_vp), _P(c_vp), c_f32, c_vp]),
    "dt_attn_workspace_bytes": (ctypes.c_int64, []),
    "dt_attn_seg_jobs_ws_fwd": (ctypes.c_int, [c_vp, c_i32, c_i32, c_i32, c_i32, c_i64, c_i64, c_i64,
                                               c_i32, _P(c_vp), _P(c_vp), _P(c_i32), _P(c_i64), c_i64, c_i64,
                                               c_i32, _P(c_i32), _P(c_i32), _P(c_i32), _P(c_i32), _P(c_i32), _P(c_i32),
                                               _P(c_vp), _P(c_vp), c_f32, c_i32, c_vp, c_i64, c_vp]),
    "dt_attn_seg_jobs_noalloc_fwd": (ctypes.c_int, [c_vp, c_i32, c_i32, c_i32, c_i32, c_i64, c_i64, c_i64,
                                                    c_i32, _P(c_vp), _P(c_vp), _P(c_i32), _P(c_i64), c_i64, c_i64,
                                                    c_i32, _P(c_i32), _P(c_i32), _P(c_i32), _P(c_i32), _P(c_i32), _P(c_i32),
                                                    _P(c_vp), _P(c_vp), c_f32, c_i32, c_vp]),
    "dt_attn_sched_seg_ws_fwd": (ctypes.c_int, [c_vp, c_i32, c_i32, c_i32, c_i32, c_i64, c_i64, c_i64,
                                                c_i32, _P(c_vp), _P(c_vp), _P(c_i32), _P(c_i64), c_i64, c_i64,
                                                c_vp, c_vp, c_i32, c_vp, c_i64, c_vp, c_i64, c_i32, c_vp, c_vp,
                                                c_i32, _P(c_i32), _P(c_i32), _P(c_i32), _P(c_i32), c_f32, c_i32,
                                                c_vp, c_i64, c_vp]),
    "dt_attn_sched_fwd": (ctypes.c_int, [c_vp, c_i32, c_i32, c_i32, c_i32, c_i64, c_i64, c_i64,
                                         c_i32, _P(c_vp), _P(c_vp), _P(c_i32), _P(c_i64), c_i64, c_i64,
                                         c_vp, c_vp, c_i32, c_vp, c_i64, c_vp, c_i64, c_i32, c_vp, c_vp,
                                         c_f32, c_vp]),
    "dt_attn_sched_seg_fwd": (ctypes.c_int, [c_vp, c_i32, c_i32, c_i32, c_i32, c_i64, c_i64, c_i64,
                                             c_i32, _P(c_vp), _P(c_vp), _P(c_i32), _P(c_i64), c_i64, c_i64,
                                             c_vp, c_vp, c_i32, c_vp, c_i64, c_vp, c_i64, c_i32, c_vp, c_vp,
                                             c_i32, _P(c_i32), _P(c_i32), _P(c_i32), _P(c_i32), c_f32, c_vp]),
    "dt_attn_varlen_jobs_fwd": (ctypes.c_int, [c_vp, c_i32, c_i32, c_i32, c_i32, c_i64, c_i64, c_i64,
                                               c_i32, _P(c_vp), _P(c_vp), _P(c_i32), _P(c_i64), c_i64, c_i64,
                                               c_i32, _P(c_i32), _P(c_i32), _P(c_i32), c_i32, c_vp, _P(c_vp), c_i32,
                                               _P(c_vp), _P(c_vp), c_f32, c_i32, c_vp]),
    "dt_attn_sched_varlen_fwd": (ctypes.c_int, [c_vp, c_i32, c_i32, c_i32, c_i32, c_i64, c_i64, c_i64,
                                                c_i32, _P(c_vp), _P(c_vp), _P(c_i32), _P(c_i64), c_i64, c_i64,
                                                c_vp, c_vp, c_i32, c_vp, c_i64, c_vp, c_i64, c_i32, c_vp, c_vp,
                                                c_i32, c_vp, _P(c_vp), c_i32, c_f32, c_i32, c_vp]),
    "dt_zero_rows_from": (ctypes.c_int, [c_vp, c_i64, c_i64, c_vp, c_vp]),
    "dt_merge_states": (ctypes.c_int, [c_i32, _P(c_vp), _P(c_vp), _P(c_i32), _P(c_i32), c_vp, c_i32, c_vp, c_i32,
                                       c_i32, c_i32, c_i32, c_i32, c_vp]),
    "dt_cache_store": (ctypes.c_int, [c_vp, c_i32, c_vp, c_i32, c_vp, c_vp, c_i32, c_i32, c_i32, c_i32, c_vp]),
    "dt_cache_load": (ctypes.c_int, [c_vp, c_vp, c_vp, c_i32, c_vp, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp]),
    "dt_state_copy": (ctypes.c_int, [c_vp, c_i32, c_vp, c_i32, c_vp, c_i32, c_vp, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp]),
    "dt_build_schedule": (ctypes.c_int, [c_vp, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp, c_vp, c_vp, c_vp]),
    "dt_build_schedule_table": (ctypes.c_int, [c_vp, c_i32, c_i32, c_i32, c_i32, c_vp, c_vp, c_vp, c_vp]),
    "dt_rel_l1_sums": (ctypes.c_int, [c_vp, c_vp, c_i64, c_vp, c_vp]),
    "dt_qk_norm_rope": (ctypes.c_int, [c_vp, c_i64, c_i64, c_i64, c_vp, c_i32, c_i32, c_i32, c_i32,
                                       c_i32, c_vp, c_vp, c_f32, c_i32, c_vp, c_vp, c_i64, c_i32, c_i32,
                                       _P(c_i32), c_i32, c_i32, c_f32, c_vp]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib: Optional[ctypes.CDLL] = None


class DitangoHipError(RuntimeError):
    pass


def load_library(path: Optional[os.PathLike] = None) -> ctypes.CDLL:
    """Load the built library (once) and declare the signatures.  Raises if it is absent."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = Path(path) if path is not None else LIB_PATH
    if not p.exists():
        raise DitangoHipError(
            f"{p} is missing: build it with `python -m ditango_amd.build` "
            "(there is no non-HIP fallback for this path)")
    lib = ctypes.CDLL(str(p))
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if path is None:
        _lib = lib
    return lib


def _check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load_library().dt_last_error().decode("utf-8", "replace")
        raise DitangoHipError(f"{what} failed with code {rc}: {msg}")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return DT_BF16
    if t.dtype == torch.float32:
        return DT_FP32
    if t.dtype == torch.float16:
        return DT_FP16
    raise DitangoHipError(f"unsupported state dtype {t.dtype} (bf16, fp16 or fp32)")


HALF_DTYPES = (torch.bfloat16, torch.float16)   # the 16-bit types the attention kernel runs in


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise DitangoHipError(msg)


def _check_qkv(q: torch.Tensor, name: str = "q", dtype: Optional[torch.dtype] = None) -> None:
    _require(q.is_cuda, f"{name} must live on the GPU")
    if dtype is None:
        _require(q.dtype in HALF_DTYPES, f"{name} must be bf16 or fp16 (got {q.dtype})")
    else:
        _require(q.dtype == dtype, f"{name} must be {dtype} like the other attention inputs (got {q.dtype})")
    _require(q.dim() == 4 and q.stride(-1) == 1, f"{name} must be [B,S,H,D] with contiguous D")


def _attn_flags(q: torch.Tensor, q_prescaled: bool) -> int:
    _require(not (q_prescaled and q.dtype == torch.float16), "a prescaled q is a bf16 mode")
    return (DT_ATTN_Q_PRESCALED if q_prescaled else 0) | (DT_ATTN_FP16 if q.dtype == torch.float16 else 0)


def lse_layout_of(lse: torch.Tensor, B: int, S: int, H: int) -> int:
    """Classify an lse tensor as [B,H,S] or [B,S,H(,1)] storage; it must be dense in that order.  Where the
    shape alone cannot tell (S == H), a 4-D tensor is read as the running layout [B,S,H,1] of utils.py:49 and a
    3-D tensor as flash-attn's [B,H,S]."""
    four_d = lse.dim() == 4 and lse.shape[-1] == 1
    if four_d:
        lse = lse.squeeze(-1)
    _require(lse.dim() == 3 and lse.dtype == torch.float32, "lse must be fp32 with 3 (or 4, last=1) dims")
    named = [((B, S, H), DT_LSE_BSH, DT_LSE_BHS), ((B, H, S), DT_LSE_BHS, DT_LSE_BSH)]
    if not four_d:
        named.reverse()
    for shape, as_is, transposed in named:
        if tuple(lse.shape) == shape:
            if lse.is_contiguous():
                return as_is
            if lse.transpose(1, 2).is_contiguous():
                return transposed
    raise DitangoHipError(f"lse of shape {tuple(lse.shape)} / strides {lse.stride()} is not a dense [B,H,S] or [B,S,H]")


# ---------------------------------------------------------------------------------------------
# K1: chunk attention
# ---------------------------------------------------------------------------------------------

def attn_chunk_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, softmax_scale: float = 0.0,
                   out: Optional[torch.Tensor] = None, lse: Optional[torch.Tensor] = None):
    """(out [B,Sq,H,D] in q's dtype -- bf16 or fp16 --, lse fp32 [B,H,Sq]) of q against one KV chunk."""
    lib = load_library()
    _check_qkv(q, "q"); _check_qkv(k, "k", q.dtype); _check_qkv(v, "v", q.dtype)
    B, Sq, H, D = q.shape
    Sk = k.shape[1]
    _require(k.shape == v.shape and k.shape[0] == B and k.shape[2] == H and k.shape[3] == D, "k/v shape mismatch")
    _require(k.stride() == v.stride(), "k and v must share strides")
    if out is None:
        out = torch.empty((B, Sq, H, D), dtype=q.dtype, device=q.device)
    if lse is None:
        lse = torch.empty((B, H, Sq), dtype=torch.float32, device=q.device)
    _require(out.is_contiguous() and lse.is_contiguous() and out.dtype == q.dtype, "out/lse must be contiguous, out in q's dtype")
    fn = lib.dt_attn_chunk_f16_fwd if q.dtype == torch.float16 else lib.dt_attn_chunk_fwd
    rc = fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
            B, Sq, Sk, H, D, q.stride(0), q.stride(1), q.stride(2),
            k.stride(0), k.stride(1), k.stride(2), float(softmax_scale), _stream())
    _check(rc, "dt_attn_chunk_fwd")
    return out, lse


def attn_chunk_f32_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, softmax_scale: float = 0.0):
    """(out fp32 [B,Sq,H,D], lse fp32 [B,H,Sq]) of fp32 q against one fp32 KV chunk, computed in fp32."""
    lib = load_library()
    for name, t in (("q", q), ("k", k), ("v", v)):
        _require(t.is_cuda and t.dtype == torch.float32 and t.dim() == 4 and t.stride(-1) == 1,
                 f"{name} must be fp32 [B,S,H,D] on the GPU with contiguous D")
    B, Sq, H, D = q.shape
    Sk = k.shape[1]
    _require(k.shape == v.shape and k.shape[0] == B and k.shape[2] == H and k.shape[3] == D, "k/v shape mismatch")
    _require(k.stride() == v.stride(), "k and v must share strides")
    out = torch.empty((B, Sq, H, D), dtype=torch.float32, device=q.device)
    lse = torch.empty((B, H, Sq), dtype=torch.float32, device=q.device)
    rc = lib.dt_attn_chunk_f32_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
                                   B, Sq, Sk, H, D, q.stride(0), q.stride(1), q.stride(2),
                                   k.stride(0), k.stride(1), k.stride(2), float(softmax_scale), _stream())
    _check(rc, "dt_attn_chunk_f32_fwd")
    return out, lse


_workspaces: "dict" = {}   # (device type, index, stream handle) -> tensor, in order of last use
MAX_WORKSPACES = 4         # streams per process that keep a workspace (about 102 MB each)


def attn_workspace(device) -> torch.Tensor:
    """The workspace of the attention launches made on the current stream of ``device`` (``dt_attn_workspace_bytes()``
    bytes).  Launches that share a workspace must be ordered on one stream; keyed by the stream, launches made on
    different streams never share one.  At most ``MAX_WORKSPACES`` streams keep theirs: the least recently used
    entry is dropped (its memory goes back to the allocator in stream order, so launches still in flight on that
    stream are safe).  The first call on a stream allocates: make it before capturing that stream in a graph --
    a workspace first created under capture would live in the graph's private pool -- or use the allocation-free
    entry point (``attn_jobs_fwd(..., no_alloc=True)``)."""
    dev = torch.device(device)
    index = dev.index if dev.index is not None else torch.cuda.current_device()
    key = (dev.type, index, torch.cuda.current_stream(index).cuda_stream)
    ws = _workspaces.pop(key, None)
    if ws is None:
        while len(_workspaces) >= MAX_WORKSPACES:
            _workspaces.pop(next(iter(_workspaces)))
        ws = torch.empty(int(load_library().dt_attn_workspace_bytes()), dtype=torch.uint8, device=dev)
    _workspaces[key] = ws       # most recently used last
    return ws


def release_workspaces() -> None:
    """Drop every attention workspace (they are re-created on demand)."""
    _workspaces.clear()


class ChunkTable:
    """Host-side table of the KV chunks one layer call can touch (pointers, lengths, strides).  A table
    may hold more chunks than one launch can address (``DT_MAX_CHUNKS``); the job launches then pass the
    sub-table of the chunks their jobs reference."""

    def __init__(self, k_chunks: Sequence[torch.Tensor], v_chunks: Sequence[torch.Tensor]):
        n = len(k_chunks)
        _require(n > 0 and n == len(v_chunks), "need at least one KV chunk and as many V as K chunks")
        self.n = n
        self.keep = (list(k_chunks), list(v_chunks))  # keep the tensors alive while pointers are in use
        self._k: List[int] = []
        self._v: List[int] = []
        self._len: List[int] = []
        self._sb: List[int] = []
        ss = sh = None
        self.dtype = k_chunks[0].dtype
        for i, (k, v) in enumerate(zip(k_chunks, v_chunks)):
            _check_qkv(k, f"k[{i}]", self.dtype); _check_qkv(v, f"v[{i}]", self.dtype)
            _require(k.shape == v.shape and k.stride() == v.stride(), f"k[{i}] / v[{i}] mismatch")
            if k.shape[1] > 0:
                if ss is None:
                    ss, sh = k.stride(1), k.stride(2)
                    self.B, self.H, self.D = k.shape[0], k.shape[2], k.shape[3]
                _require((k.stride(1), k.stride(2)) == (ss, sh), "all chunks must share token/head strides")
                _require((k.shape[0], k.shape[2], k.shape[3]) == (self.B, self.H, self.D), "chunk B/H/D mismatch")
            self._k.append(k.data_ptr())
            self._v.append(v.data_ptr())
            self._len.append(k.shape[1])
            self._sb.append(k.stride(0))
        _require(ss is not None, "all KV chunks are empty")
        self.ss, self.sh = ss, sh
        self._whole = self.arrays(range(n)) if n <= DT_MAX_CHUNKS else None

    def arrays(self, ids: Sequence[int]):
        """ctypes arrays (k_ptrs, v_ptrs, lens, batch strides) of the chunks ``ids``, in that order."""
        ids = list(ids)
        m = len(ids)
        _require(0 < m <= DT_MAX_CHUNKS, f"one launch addresses 1..{DT_MAX_CHUNKS} KV chunks, not {m}")
        return ((c_vp * m)(*[self._k[i] for i in ids]), (c_vp * m)(*[self._v[i] for i in ids]),
                (c_i32 * m)(*[self._len[i] for i in ids]), (c_i64 * m)(*[self._sb[i] for i in ids]))

    def whole(self):
        """The arrays of all chunks (tables that fit one launch)."""
        _require(self._whole is not None, f"the table holds {self.n} chunks, one launch addresses {DT_MAX_CHUNKS}")
        return self._whole

    # the whole-table arrays under their old names
    @property
    def k_ptrs(self):
        return self.whole()[0]

    @property
    def v_ptrs(self):
        return self.whole()[1]

    @property
    def lens(self):
        return self.whole()[2]

    @property
    def sb(self):
        return self.whole()[3]


class DeviceSegments:
    """Segment boundaries of a packed variable-length batch that live in device memory, as
    ``flash_attn_varlen_func`` takes them: ``cu_q`` int32 ``[n_seg + 1]`` for the queries and one such tensor
    per KV chunk for its keys (``cu_kv[c]``; ``None`` for a chunk without keys).  ``max_seqlen_q`` is the
    host-side upper bound of a segment's length that sizes the grid.  Nothing here reads device memory."""

    def __init__(self, cu_q: torch.Tensor, cu_kv: Sequence[Optional[torch.Tensor]], max_seqlen_q: int):
        for name, t in [("cu_seqlens_q", cu_q)] + [(f"cu_seqlens_kv[{i}]", t) for i, t in enumerate(cu_kv) if t is not None]:
            _require(torch.is_tensor(t) and t.is_cuda and t.dtype == torch.int32 and t.dim() == 1 and t.is_contiguous(),
                     f"{name} must be a contiguous int32 vector on the GPU")
            _require(t.numel() == cu_q.numel(), f"{name} must have as many entries as cu_seqlens_q")
        _require(cu_q.numel() >= 2, "cu_seqlens_q needs at least two entries")
        _require(int(max_seqlen_q) > 0, "max_seqlen_q must be positive")
        self.cu_q = cu_q
        self.cu_kv = list(cu_kv)
        self.n_seg = cu_q.numel() - 1
        self.max_seqlen_q = int(max_seqlen_q)

    def kv_pointers(self, ids: Sequence[int]):
        ids = list(ids)
        return (c_vp * len(ids))(*[self.cu_kv[i].data_ptr() if self.cu_kv[i] is not None else None for i in ids])

    def window(self, w0: int, w1: int) -> "DeviceSegments":
        return DeviceSegments(self.cu_q, self.cu_kv[w0:w1], self.max_seqlen_q)


def attn_jobs_fwd(q: torch.Tensor, table: ChunkTable, jobs: Sequence[Sequence[int]],
                  outs: Sequence[torch.Tensor], lses: Sequence[torch.Tensor], softmax_scale: float = 0.0,
                  q_ranges: Optional[Sequence[Tuple[int, int]]] = None,
                  kv_ranges: Optional[Sequence[Sequence[Tuple[int, int]]]] = None,
                  workspace: Optional[torch.Tensor] = None, q_prescaled: bool = False,
                  no_alloc: bool = False, dev_segments: Optional["DeviceSegments"] = None,
                  job_segments: Optional[Sequence[int]] = None) -> None:
    """One launch; job j attends q to the concatenation of chunks ``jobs[j]`` and writes (outs[j], lses[j]).

    ``q_ranges[j] = (begin, length)`` restricts job j to those query rows (the rest of its
    destination is left untouched); ``kv_ranges[j][i] = (begin, length)`` restricts the i-th chunk
    of job j to those keys.  Several jobs may share one destination if their rows are disjoint
    (the segments of a packed variable-length batch).  Launches are split to respect the limits
    of one launch.  With a ``workspace`` (``attn_workspace(device)``) the last, partly filled round of
    workgroups of a launch is split along the keys and folded back (tail balancing).
    ``q_prescaled``: q already carries ``softmax_scale * log2(e)`` (folded in before its rounding to
    bf16); ``softmax_scale`` is then ignored and the softmax is that of ``q k^T * ln 2``.
    ``no_alloc``: go through ``dt_attn_seg_jobs_noalloc_fwd``, which splits the tail inside the library's
    own device array instead of a workspace (for callers that cannot allocate).
    ``dev_segments`` with ``job_segments``: the segment boundaries stay in device memory
    (``dt_attn_varlen_jobs_fwd``); job j is segment ``job_segments[j]`` of its state and the host reads none
    of the boundaries."""
    lib = load_library()
    _check_qkv(q, "q", table.dtype)
    flags = _attn_flags(q, q_prescaled)
    B, Sq, H, D = q.shape
    _require((B, H, D) == (table.B, table.H, table.D), "q and KV chunks disagree on B/H/D")
    _require(not (no_alloc and workspace is not None), "no_alloc launches take no workspace")
    nj = len(jobs)
    if dev_segments is not None:
        _require(q_ranges is None and kv_ranges is None and not no_alloc, "device segment boundaries replace the host ranges")
        _require(job_segments is not None and len(job_segments) == nj, "one segment index per job")
        _require(len(dev_segments.cu_kv) == table.n, "one cu_seqlens_kv per chunk of the table")
    _require(nj == len(outs) == len(lses), "one destination per job")
    _require(q_ranges is None or len(q_ranges) == nj, "one query range per job")
    _require(kv_ranges is None or len(kv_ranges) == nj, "one list of key ranges per job")
    for j in range(nj):
        o, l = outs[j], lses[j]
        _require(o.dtype == q.dtype and o.is_contiguous() and tuple(o.shape) == (B, Sq, H, D), f"outs[{j}] must be contiguous [B,Sq,H,D] in q's dtype")
        _require(l.dtype == torch.float32 and l.is_contiguous() and tuple(l.shape) == (B, H, Sq), f"lses[{j}] must be contiguous fp32 [B,H,Sq]")
        _require(len(jobs[j]) <= DT_MAX_JOB_ENTRIES, f"job {j} references more than {DT_MAX_JOB_ENTRIES} chunks")
    # split into launches that fit the per-launch limits (jobs, chunk references, distinct chunks)
    start = 0
    while start < nj:
        end, entries = start, 0
        used = set()
        while end < nj and end - start < DT_MAX_JOBS and entries + len(jobs[end]) <= DT_MAX_JOB_ENTRIES:
            more = used | {int(c) for c in jobs[end]}
            if table.n > DT_MAX_CHUNKS and len(more) > DT_MAX_CHUNKS:
                break
            used = more
            entries += len(jobs[end])
            end += 1
        _require(end > start, f"job {start} references more than {DT_MAX_CHUNKS} distinct chunks: split it and merge the parts")
        n = end - start
        if table.n <= DT_MAX_CHUNKS:
            t_k, t_v, t_len, t_sb = table.whole()
            t_n = table.n
            local = None
        else:
            ids = sorted(used) or [0]
            t_k, t_v, t_len, t_sb = table.arrays(ids)
            t_n = len(ids)
            local = {c: i for i, c in enumerate(ids)}
        begin = (c_i32 * (n + 1))()
        flat: List[int] = []
        kvb: List[int] = []
        kvl: List[int] = []
        for jj in range(n):
            j = start + jj
            begin[jj] = len(flat)
            for i, c in enumerate(jobs[j]):
                c = int(c)
                _require(0 <= c < table.n, f"job {j} references chunk {c} outside the table of {table.n}")
                flat.append(c if local is None else local[c])
                if kv_ranges is not None:
                    kvb.append(int(kv_ranges[j][i][0]))
                    kvl.append(int(kv_ranges[j][i][1]))
        begin[n] = len(flat)
        m = max(1, len(flat))
        chunks = (c_i32 * m)(*flat)
        a_kvb = (c_i32 * m)(*kvb) if kv_ranges is not None else None
        a_kvl = (c_i32 * m)(*kvl) if kv_ranges is not None else None
        a_qb = (c_i32 * n)(*[int(q_ranges[start + jj][0]) for jj in range(n)]) if q_ranges is not None else None
        a_ql = (c_i32 * n)(*[int(q_ranges[start + jj][1]) for jj in range(n)]) if q_ranges is not None else None
        out_ptrs = (c_vp * n)(*[outs[start + jj].data_ptr() for jj in range(n)])
        lse_ptrs = (c_vp * n)(*[lses[start + jj].data_ptr() for jj in range(n)])
        if dev_segments is not None:
            seg_ids = (c_i32 * n)(*[int(job_segments[start + jj]) for jj in range(n)])
            cu_kv = dev_segments.kv_pointers(range(table.n) if local is None else ids)
            rc = lib.dt_attn_varlen_jobs_fwd(q.data_ptr(), B, Sq, H, D, q.stride(0), q.stride(1), q.stride(2),
                                             t_n, t_k, t_v, t_len, t_sb, table.ss, table.sh,
                                             n, begin, chunks, seg_ids, dev_segments.n_seg, dev_segments.cu_q.data_ptr(),
                                             cu_kv, int(dev_segments.max_seqlen_q), out_ptrs, lse_ptrs,
                                             float(softmax_scale), flags, _stream())
            _check(rc, "dt_attn_varlen_jobs_fwd")
        elif no_alloc:
            rc = lib.dt_attn_seg_jobs_noalloc_fwd(q.data_ptr(), B, Sq, H, D, q.stride(0), q.stride(1), q.stride(2),
                                                  t_n, t_k, t_v, t_len, t_sb, table.ss, table.sh,
                                                  n, begin, chunks, a_kvb, a_kvl, a_qb, a_ql, out_ptrs,
                                                  lse_ptrs, float(softmax_scale), flags, _stream())
            _check(rc, "dt_attn_seg_jobs_noalloc_fwd")
        else:
            rc = lib.dt_attn_seg_jobs_ws_fwd(q.data_ptr(), B, Sq, H, D, q.stride(0), q.stride(1), q.stride(2),
                                             t_n, t_k, t_v, t_len, t_sb, table.ss, table.sh,
                                             n, begin, chunks, a_kvb, a_kvl, a_qb, a_ql, out_ptrs, lse_ptrs,
                                             float(softmax_scale), flags,
                                             workspace.data_ptr() if workspace is not None else None,
                                             workspace.numel() * workspace.element_size() if workspace is not None else 0,
                                             _stream())
            _check(rc, "dt_attn_seg_jobs_ws_fwd")
        start = end


def attn_sched_fwd(q: torch.Tensor, table: ChunkTable, dev_compute_ids: torch.Tensor, dev_count: torch.Tensor,
                   max_jobs: int, slot_out: torch.Tensor, slot_lse: torch.Tensor, diag: int,
                   diag_out: Optional[torch.Tensor], diag_lse: Optional[torch.Tensor],
                   softmax_scale: float = 0.0, seg_q: Optional[Sequence[Tuple[int, int]]] = None,
                   seg_kv: Optional[Sequence[Sequence[Tuple[int, int]]]] = None,
                   workspace: Optional[torch.Tensor] = None, q_prescaled: bool = False,
                   dev_segments: Optional[DeviceSegments] = None) -> None:
    """Device-scheduled launch: chunk ids come from ``dev_compute_ids[:dev_count]`` in device memory and
    each state lands in its slot of the arena (``slot_out [C,B,Sq,H,D]`` in q's dtype, ``slot_lse [C,B,H,Sq]`` fp32).

    On a packed variable-length batch, ``seg_q[s] = (begin, length)`` are the query rows of segment s and
    ``seg_kv[c][s] = (begin, length)`` its keys inside chunk c; every scheduled chunk then runs once per segment."""
    lib = load_library()
    _check_qkv(q, "q", table.dtype)
    flags = _attn_flags(q, q_prescaled)
    B, Sq, H, D = q.shape
    _require((B, H, D) == (table.B, table.H, table.D), "q and KV chunks disagree on B/H/D")
    _require(dev_compute_ids.dtype == torch.int32 and dev_count.dtype == torch.int32 and dev_compute_ids.is_cuda and dev_count.is_cuda,
             "schedule tensors must be int32 on the GPU")
    _require(dev_compute_ids.is_contiguous() and dev_compute_ids.numel() >= max_jobs, "compute id list shorter than max_jobs")
    _require(slot_out.dtype == q.dtype and slot_out.is_contiguous() and tuple(slot_out.shape[1:]) == (B, Sq, H, D)
             and slot_out.shape[0] >= table.n, "slot_out must be contiguous [C,B,Sq,H,D] in q's dtype")
    _require(slot_lse.dtype == torch.float32 and slot_lse.is_contiguous() and tuple(slot_lse.shape[1:]) == (B, H, Sq)
             and slot_lse.shape[0] >= table.n, "slot_lse must be contiguous fp32 [C,B,H,Sq]")
    if 0 <= diag < table.n:
        _require(diag_out is not None and diag_lse is not None, "a diag chunk needs (diag_out, diag_lse)")
        _require(diag_out.dtype == q.dtype and diag_out.is_contiguous() and tuple(diag_out.shape) == (B, Sq, H, D), "diag_out must be contiguous [B,Sq,H,D] in q's dtype")
        _require(diag_lse.dtype == torch.float32 and diag_lse.is_contiguous() and tuple(diag_lse.shape) == (B, H, Sq), "diag_lse must be contiguous fp32 [B,H,Sq]")
    if dev_segments is not None:
        # segment boundaries in device memory: every scheduled chunk runs once per segment, the host reads nothing
        _require(seg_q is None and seg_kv is None, "device segment boundaries replace the host ranges")
        _require(len(dev_segments.cu_kv) == table.n, "one cu_seqlens_kv per chunk of the table")
        rc = lib.dt_attn_sched_varlen_fwd(q.data_ptr(), B, Sq, H, D, q.stride(0), q.stride(1), q.stride(2),
                                          table.n, table.k_ptrs, table.v_ptrs, table.lens, table.sb, table.ss, table.sh,
                                          dev_compute_ids.data_ptr(), dev_count.data_ptr(), int(max_jobs),
                                          slot_out.data_ptr(), slot_out.stride(0), slot_lse.data_ptr(), slot_lse.stride(0),
                                          int(diag), diag_out.data_ptr() if diag_out is not None else None,
                                          diag_lse.data_ptr() if diag_lse is not None else None,
                                          dev_segments.n_seg, dev_segments.cu_q.data_ptr(),
                                          dev_segments.kv_pointers(range(table.n)), dev_segments.max_seqlen_q,
                                          float(softmax_scale), flags, _stream())
        _check(rc, "dt_attn_sched_varlen_fwd")
        return
    n_seg, a_qb, a_ql, a_kb, a_kl = 0, None, None, None, None
    if seg_q is not None:
        n_seg = len(seg_q)
        _require(seg_kv is not None and len(seg_kv) == table.n and all(len(r) == n_seg for r in seg_kv),
                 "seg_kv needs one (begin, length) per chunk and segment")
        _require(0 < n_seg <= DT_MAX_SEGMENTS and n_seg * table.n <= DT_MAX_JOB_ENTRIES,
                 f"need 1..{DT_MAX_SEGMENTS} segments and at most {DT_MAX_JOB_ENTRIES} (chunk, segment) pairs")
        a_qb = (c_i32 * n_seg)(*[int(b) for b, _ in seg_q])
        a_ql = (c_i32 * n_seg)(*[int(n) for _, n in seg_q])
        a_kb = (c_i32 * (n_seg * table.n))(*[int(b) for row in seg_kv for b, _ in row])
        a_kl = (c_i32 * (n_seg * table.n))(*[int(n) for row in seg_kv for _, n in row])
    rc = lib.dt_attn_sched_seg_ws_fwd(q.data_ptr(), B, Sq, H, D, q.stride(0), q.stride(1), q.stride(2),
                                   table.n, table.k_ptrs, table.v_ptrs, table.lens, table.sb, table.ss, table.sh,
                                   dev_compute_ids.data_ptr(), dev_count.data_ptr(), int(max_jobs),
                                   slot_out.data_ptr(), slot_out.stride(0), slot_lse.data_ptr(), slot_lse.stride(0),
                                   int(diag), diag_out.data_ptr() if diag_out is not None else None,
                                   diag_lse.data_ptr() if diag_lse is not None else None,
                                   n_seg, a_qb, a_ql, a_kb, a_kl, float(softmax_scale), flags,
                                   workspace.data_ptr() if workspace is not None else None,
                                   workspace.numel() * workspace.element_size() if workspace is not None else 0, _stream())
    _check(rc, "dt_attn_sched_seg_ws_fwd")


# ---------------------------------------------------------------------------------------------
# K2: merge, K3: cache store/load
# ---------------------------------------------------------------------------------------------

def _merge_once(outs, lses, dst_out, dst_lse, B, Sq, H, D) -> None:
    lib = load_library()
    n = len(outs)
    out_ptrs = (c_vp * n)()
    lse_ptrs = (c_vp * n)()
    dts = (c_i32 * n)()
    lays = (c_i32 * n)()
    for i, (o, l) in enumerate(zip(outs, lses)):
        _require(o.is_cuda and o.is_contiguous() and tuple(o.shape) == (B, Sq, H, D), f"outs[{i}] must be contiguous [B,Sq,H,D] on the GPU")
        out_ptrs[i] = o.data_ptr()
        lse_ptrs[i] = l.data_ptr()
        dts[i] = _dtype_code(o)
        lays[i] = lse_layout_of(l, B, Sq, H)
    dlay = lse_layout_of(dst_lse, B, Sq, H)
    rc = lib.dt_merge_states(n, out_ptrs, lse_ptrs, dts, lays, dst_out.data_ptr(), _dtype_code(dst_out),
                             dst_lse.data_ptr(), dlay, B, Sq, H, D, _stream())
    _check(rc, "dt_merge_states")


def merge_states(outs: Sequence[torch.Tensor], lses: Sequence[torch.Tensor],
                 dst_out: Optional[torch.Tensor] = None, dst_lse: Optional[torch.Tensor] = None,
                 dst_dtype: torch.dtype = torch.float32, dst_lse_bsh: bool = False):
    """N-way LSE merge.  outs[i] contiguous [B,Sq,H,D] (bf16, fp16 or fp32, in any mix), lses[i] fp32 in
    [B,H,Sq] or [B,Sq,H(,1)] storage.  Returns (dst_out, dst_lse).  Up to ``DT_MAX_MERGE`` states are one
    pass over HBM; more are folded in rounds through a running fp32 state that is updated in place (the
    merge is associative; the running state is never rounded below fp32)."""
    n = len(outs)
    _require(n > 0 and n == len(lses), "need at least one state and one lse per state")
    B, Sq, H, D = outs[0].shape
    dev = outs[0].device
    if dst_out is None:
        dst_out = torch.empty((B, Sq, H, D), dtype=dst_dtype, device=dev)
    if dst_lse is None:
        dst_lse = torch.empty((B, Sq, H, 1) if dst_lse_bsh else (B, H, Sq), dtype=torch.float32, device=dev)
    _require(dst_out.is_contiguous() and tuple(dst_out.shape) == (B, Sq, H, D), "dst_out must be contiguous [B,Sq,H,D]")
    outs, lses = list(outs), list(lses)
    if n > DT_MAX_MERGE:
        run_out = torch.empty((B, Sq, H, D), dtype=torch.float32, device=dev)
        run_lse = torch.empty((B, H, Sq), dtype=torch.float32, device=dev)
        _merge_once(outs[:DT_MAX_MERGE], lses[:DT_MAX_MERGE], run_out, run_lse, B, Sq, H, D)
        i = DT_MAX_MERGE
        while n - i > DT_MAX_MERGE - 1:
            _merge_once([run_out] + outs[i:i + DT_MAX_MERGE - 1], [run_lse] + lses[i:i + DT_MAX_MERGE - 1],
                        run_out, run_lse, B, Sq, H, D)
            i += DT_MAX_MERGE - 1
        outs, lses = [run_out] + outs[i:], [run_lse] + lses[i:]
    _merge_once(outs, lses, dst_out, dst_lse, B, Sq, H, D)
    return dst_out, dst_lse


def cache_store(src_out: torch.Tensor, src_lse: torch.Tensor, slot_out: torch.Tensor, slot_lse: torch.Tensor) -> None:
    lib = load_library()
    B, Sq, H, D = src_out.shape
    _require(src_out.is_cuda and src_out.is_contiguous(), "src_out must be contiguous on the GPU")
    _require(slot_out.dtype in HALF_DTYPES and slot_out.is_contiguous() and tuple(slot_out.shape) == (B, Sq, H, D), "slot_out must be contiguous bf16 or fp16 [B,Sq,H,D]")
    _require(slot_lse.dtype == torch.float32 and slot_lse.is_contiguous() and tuple(slot_lse.shape) == (B, H, Sq), "slot_lse must be contiguous fp32 [B,H,Sq]")
    if slot_out.dtype == torch.bfloat16:
        rc = lib.dt_cache_store(src_out.data_ptr(), _dtype_code(src_out), src_lse.data_ptr(), lse_layout_of(src_lse, B, Sq, H),
                                slot_out.data_ptr(), slot_lse.data_ptr(), B, Sq, H, D, _stream())
    else:   # fp16 slots of a model that runs in fp16
        rc = lib.dt_state_copy(src_out.data_ptr(), _dtype_code(src_out), src_lse.data_ptr(), lse_layout_of(src_lse, B, Sq, H),
                               slot_out.data_ptr(), DT_FP16, slot_lse.data_ptr(), DT_LSE_BHS, B, Sq, H, D, _stream())
    _check(rc, "dt_cache_store")


def cache_load(slot_out: torch.Tensor, slot_lse: torch.Tensor, dst_dtype: torch.dtype = torch.float32,
               dst_lse_bsh: bool = False, dst_out: Optional[torch.Tensor] = None, dst_lse: Optional[torch.Tensor] = None):
    lib = load_library()
    B, Sq, H, D = slot_out.shape
    _require(slot_out.dtype in HALF_DTYPES and slot_out.is_contiguous(), "slot_out must be contiguous bf16 or fp16")
    _require(slot_lse.dtype == torch.float32 and slot_lse.is_contiguous() and tuple(slot_lse.shape) == (B, H, Sq), "slot_lse must be contiguous fp32 [B,H,Sq]")
    if dst_out is None:
        dst_out = torch.empty((B, Sq, H, D), dtype=dst_dtype, device=slot_out.device)
    if dst_lse is None:
        dst_lse = torch.empty((B, Sq, H, 1) if dst_lse_bsh else (B, H, Sq), dtype=torch.float32, device=slot_out.device)
    _require(dst_out.is_contiguous() and tuple(dst_out.shape) == (B, Sq, H, D), "dst_out must be contiguous [B,Sq,H,D]")
    dst_lse_bsh = lse_layout_of(dst_lse, B, Sq, H) == DT_LSE_BSH
    if slot_out.dtype == torch.bfloat16:
        rc = lib.dt_cache_load(slot_out.data_ptr(), slot_lse.data_ptr(), dst_out.data_ptr(), _dtype_code(dst_out),
                               dst_lse.data_ptr(), DT_LSE_BSH if dst_lse_bsh else DT_LSE_BHS, B, Sq, H, D, _stream())
    else:
        rc = lib.dt_state_copy(slot_out.data_ptr(), DT_FP16, slot_lse.data_ptr(), DT_LSE_BHS, dst_out.data_ptr(),
                               _dtype_code(dst_out), dst_lse.data_ptr(), DT_LSE_BSH if dst_lse_bsh else DT_LSE_BHS,
                               B, Sq, H, D, _stream())
    _check(rc, "dt_cache_load")
    return dst_out, dst_lse


def zero_rows_from(t: torch.Tensor, first_row: torch.Tensor) -> None:
    """Zero the rows ``[first_row[0], n)`` of ``t`` (contiguous, rows along dim 0), the index read on the device."""
    lib = load_library()
    _require(t.is_cuda and t.is_contiguous() and t.dim() >= 1, "t must be a contiguous device tensor")
    _require(first_row.is_cuda and first_row.dtype == torch.int32 and first_row.numel() >= 1, "first_row must be int32 on the GPU")
    n = t.shape[0]
    row_bytes = (t.numel() // max(n, 1)) * t.element_size()
    rc = lib.dt_zero_rows_from(t.data_ptr(), n, row_bytes, first_row.data_ptr(), _stream())
    _check(rc, "dt_zero_rows_from")


# ---------------------------------------------------------------------------------------------
# K4: schedule builder, rel-L1 sums
# ---------------------------------------------------------------------------------------------

def build_schedule(mask: torch.Tensor, t: int, l: int, diag: int = -1):
    """(compute_ids [C], reuse_ids [C], counts [2]) int32 device tensors for row (t, l) of mask uint8 [T,L,C]."""
    lib = load_library()
    _require(mask.is_cuda and mask.dtype == torch.uint8 and mask.dim() == 3 and mask.is_contiguous(), "mask must be contiguous uint8 [T,L,C] on the GPU")
    T, L, C = mask.shape
    comp = torch.empty(C, dtype=torch.int32, device=mask.device)
    reu = torch.empty(C, dtype=torch.int32, device=mask.device)
    cnt = torch.empty(2, dtype=torch.int32, device=mask.device)
    rc = lib.dt_build_schedule(mask.data_ptr(), T, L, C, int(t), int(l), int(diag), comp.data_ptr(), reu.data_ptr(), cnt.data_ptr(), _stream())
    _check(rc, "dt_build_schedule")
    return comp, reu, cnt


def build_schedule_table(mask: torch.Tensor, diag: int = -1):
    lib = load_library()
    _require(mask.is_cuda and mask.dtype == torch.uint8 and mask.dim() == 3 and mask.is_contiguous(), "mask must be contiguous uint8 [T,L,C] on the GPU")
    T, L, C = mask.shape
    comp = torch.empty((T, L, C), dtype=torch.int32, device=mask.device)
    reu = torch.empty((T, L, C), dtype=torch.int32, device=mask.device)
    cnt = torch.empty((T, L, 2), dtype=torch.int32, device=mask.device)
    rc = lib.dt_build_schedule_table(mask.data_ptr(), T, L, C, int(diag), comp.data_ptr(), reu.data_ptr(), cnt.data_ptr(), _stream())
    _check(rc, "dt_build_schedule_table")
    return comp, reu, cnt


def rel_l1_sums(a: torch.Tensor, b: torch.Tensor, sums: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp64 [4] device tensor: sum|a-b|, sum|a|, sum|b|, count over entries where neither is NaN (no host sync)."""
    lib = load_library()
    _require(a.is_cuda and b.is_cuda and a.dtype == torch.float32 and b.dtype == torch.float32, "inputs must be fp32 on the GPU")
    _require(a.is_contiguous() and b.is_contiguous() and a.numel() == b.numel(), "inputs must be contiguous and equally sized")
    if sums is None:
        sums = torch.zeros(4, dtype=torch.float64, device=a.device)
    rc = lib.dt_rel_l1_sums(a.data_ptr(), b.data_ptr(), a.numel(), sums.data_ptr(), _stream())
    _check(rc, "dt_rel_l1_sums")
    return sums


def qk_norm_rope(x: torch.Tensor, *, norm: int = DT_NORM_NONE, weight: Optional[torch.Tensor] = None,
                 bias: Optional[torch.Tensor] = None, eps: float = 1e-6, rope: int = DT_ROPE_NONE,
                 cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None,
                 rope_begin: int = 0, rope_end: Optional[int] = None, sections: Sequence[int] = (),
                 rounding: int = 0, out: Optional[torch.Tensor] = None, out_scale: float = 1.0) -> torch.Tensor:
    """x bf16 or fp16 ``[B,S,H,D]`` (any strides with a contiguous last dimension) -> ``[B,S,H,D]`` contiguous in
    the same dtype, normalised over D and rotated on token rows ``[rope_begin, rope_end)``.  cos/sin are fp32
    ``[rope_end-rope_begin, D]`` or ``[B, rope_end-rope_begin, D]``.  ``out_scale`` multiplies the result
    before its rounding to the output dtype; the ``DT_ROUND_*`` bits round to x's dtype."""
    lib = load_library()
    _require(x.is_cuda and x.dtype in HALF_DTYPES and x.dim() == 4 and x.stride(3) == 1, "x must be bf16 or fp16 [B,S,H,D] on the GPU")
    B, S, H, D = x.shape
    if out is None:
        out = torch.empty((B, S, H, D), dtype=x.dtype, device=x.device)
    _require(out.is_cuda and out.dtype == x.dtype and out.is_contiguous() and tuple(out.shape) == (B, S, H, D),
             "out must be a contiguous [B,S,H,D] in x's dtype")
    rounding = int(rounding) | (DT_IO_FP16 if x.dtype == torch.float16 else 0)
    for name, t in (("weight", weight), ("bias", bias)):
        _require(t is None or (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.numel() == D),
                 f"{name} must be fp32 [D] on the GPU")
    if rope_end is None:
        rope_end = S
    tab_sb = 0
    if rope != DT_ROPE_NONE and rope_end > rope_begin:
        rows = rope_end - rope_begin
        for name, t in (("cos", cos), ("sin", sin)):
            _require(t is not None and t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()
                     and t.shape[-1] == D and t.shape[-2] == rows and t.dim() in (2, 3),
                     f"{name} must be a contiguous fp32 [rows, D] or [B, rows, D] table on the GPU")
        _require(cos.shape == sin.shape, "cos and sin must have one shape")
        if cos.dim() == 3:
            _require(cos.shape[0] == B, "batched tables need B leading entries")
            tab_sb = rows * D
    sec = (c_i32 * max(1, len(sections)))(*[int(v) for v in sections])
    rc = lib.dt_qk_norm_rope(x.data_ptr(), x.stride(0), x.stride(1), x.stride(2), out.data_ptr(), B, S, H, D,
                             int(norm), weight.data_ptr() if weight is not None else None,
                             bias.data_ptr() if bias is not None else None, float(eps), int(rope),
                             cos.data_ptr() if cos is not None else None, sin.data_ptr() if sin is not None else None,
                             tab_sb, int(rope_begin), int(rope_end), sec, len(sections), int(rounding), float(out_scale),
                             _stream())
    _check(rc, "dt_qk_norm_rope")
    return out
