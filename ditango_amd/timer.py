"""Named wall timers with the reference's surface (timer.py:1-141):
``get_timer(name)`` is a context manager / decorator that synchronises the GPU on
entry and exit when timing is enabled and costs nothing when it is not (the
reference enables it from denoise step 2 on)."""
import time
from contextlib import ContextDecorator
from typing import Dict, List

import torch

_ENABLED = False
_RECORDS: Dict[str, List[float]] = {}


def init_timer(enable: bool = True) -> None:
    global _ENABLED
    _ENABLED = bool(enable)
    _RECORDS.clear()


def enable_timing() -> None:
    global _ENABLED
    _ENABLED = True


def disable_timing() -> None:
    global _ENABLED
    _ENABLED = False


def is_timing_enabled() -> bool:
    return _ENABLED


class _Timer(ContextDecorator):
    def __init__(self, name: str):
        self.name = name
        self._t0 = None

    def __enter__(self):
        if _ENABLED:
            if torch.cuda.is_available():
                torch.cuda.synchronize()
            self._t0 = time.perf_counter()
        return self

    def __exit__(self, *exc):
        if _ENABLED and self._t0 is not None:
            if torch.cuda.is_available():
                torch.cuda.synchronize()
            _RECORDS.setdefault(self.name, []).append(time.perf_counter() - self._t0)
            self._t0 = None
        return False


def get_timer(name: str) -> _Timer:
    return _Timer(name)


def get_time_statistics() -> Dict[str, Dict[str, float]]:
    out = {}
    for name, xs in _RECORDS.items():
        if xs:
            out[name] = {"count": len(xs), "min_ms": 1e3 * min(xs), "max_ms": 1e3 * max(xs), "avg_ms": 1e3 * sum(xs) / len(xs)}
    return out


def print_time_statistics() -> None:
    for name, st in get_time_statistics().items():
        print(f"{name:>16s}: n={st['count']:5d} min={st['min_ms']:.3f} ms max={st['max_ms']:.3f} ms avg={st['avg_ms']:.3f} ms", flush=True)
