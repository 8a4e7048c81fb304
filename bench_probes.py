"""ctypes binding of ``libditango_probes.so`` (``include/ditango_probes.h``): the three micro-benchmarks
``bench.py`` prints next to the nominal peaks.  They are measurement aids, not part of the drop-in library;
nothing under ``ditango_amd/`` imports this module."""
from __future__ import annotations

import ctypes
from pathlib import Path
from typing import Optional, Sequence

import torch

PROBES_PATH = Path(__file__).resolve().parent / "ditango_amd" / "lib" / "libditango_probes.so"
DTP_MAX_STREAMS = 64

c_i32, c_i64, c_vp = ctypes.c_int32, ctypes.c_int64, ctypes.c_void_p
_SIGNATURES = {
    "dtp_last_error": (ctypes.c_char_p, []),
    "dtp_hbm_read_probe": (ctypes.c_int, [ctypes.POINTER(c_vp), c_i32, c_i64, c_vp, c_vp]),
    "dtp_mfma_probe": (ctypes.c_int, [c_i32, c_i32, c_vp, c_vp]),
    "dtp_coissue_probe": (ctypes.c_int, [c_i32, c_i32, c_i32, c_i32, c_vp, c_vp]),
    "dtp_empty_launch": (ctypes.c_int, [c_i32, c_i32, c_vp]),
}
EXPORTED_SYMBOLS = tuple(_SIGNATURES)
_lib: Optional[ctypes.CDLL] = None


class ProbeError(RuntimeError):
    pass


def load_library() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not PROBES_PATH.exists():
            raise ProbeError(f"{PROBES_PATH} is missing: build it with `python -m ditango_amd.build`")
        lib = ctypes.CDLL(str(PROBES_PATH))
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise ProbeError(f"{what} failed with code {rc}: {load_library().dtp_last_error().decode('utf-8', 'replace')}")


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise ProbeError(msg)


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def hbm_read_probe(buffers: Sequence[torch.Tensor], sink: torch.Tensor) -> None:
    """Read ``buffers`` (equally sized, contiguous, a multiple of 256 bytes each) with the merge kernel's
    access pattern and discard the data: the bandwidth yardstick of the HBM-bound kernels."""
    lib = load_library()
    n = len(buffers)
    nbytes = buffers[0].numel() * buffers[0].element_size()
    for b in buffers:
        _require(b.is_cuda and b.is_contiguous() and b.numel() * b.element_size() == nbytes,
                 "probe buffers must be equally sized contiguous device tensors")
    _require(sink.is_cuda and sink.numel() * sink.element_size() >= 4, "sink must be a device tensor of at least 4 bytes")
    ptrs = (c_vp * n)(*[b.data_ptr() for b in buffers])
    _check(lib.dtp_hbm_read_probe(ptrs, n, nbytes // 256 * 256, sink.data_ptr(), _stream()), "dtp_hbm_read_probe")


def mfma_probe(workgroups: int, iters: int, sink: torch.Tensor) -> float:
    """Launch the register-only MFMA loop and return the FLOP the launch performs:
    ``workgroups * 8`` wavefronts x ``4 * iters`` bf16 MFMAs of 32 x 32 x 16."""
    lib = load_library()
    _require(sink.is_cuda and sink.numel() * sink.element_size() >= 4, "sink must be a device tensor of at least 4 bytes")
    _check(lib.dtp_mfma_probe(int(workgroups), int(iters), sink.data_ptr(), _stream()), "dtp_mfma_probe")
    return float(workgroups) * 8 * 4 * iters * 32768.0


def coissue_probe(workgroups: int, iters: int, head_dim: int, with_softmax: bool, sink: torch.Tensor) -> float:
    """Launch the co-issue probe (one wavefront of each SIMD issues MFMAs; with ``with_softmax`` the other one
    issues the softmax's vector instructions per MFMA at that head dimension) and return the FLOP of the
    launch: ``workgroups * 4`` wavefronts x ``4 * iters`` bf16 MFMAs of 32 x 32 x 16."""
    lib = load_library()
    _require(sink.is_cuda and sink.numel() * sink.element_size() >= 4, "sink must be a device tensor of at least 4 bytes")
    _check(lib.dtp_coissue_probe(int(workgroups), int(iters), int(head_dim), int(bool(with_softmax)), sink.data_ptr(),
                                 _stream()), "dtp_coissue_probe")
    return float(workgroups) * 4 * 4 * iters * 32768.0


def empty_launch(workgroups: int, threads: int) -> None:
    """Launch a kernel of that grid that does nothing (the floor of a launch)."""
    _check(load_library().dtp_empty_launch(int(workgroups), int(threads), _stream()), "dtp_empty_launch")
