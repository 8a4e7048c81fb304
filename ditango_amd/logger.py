"""Logging shim with the reference's entry point (logger.py:1-95): ``init_logger(name)``.

Level from ``LOG_LEVEL`` (default ``info`` here; the reference defaults to debug),
optional per-process file under ``LOG_DIR``.
"""
import logging
import os
import sys

_FORMAT = "%(levelname)s %(asctime)s [%(name)s:%(lineno)d] %(message)s"
_configured = False


def _configure_root() -> None:
    global _configured
    if _configured:
        return
    root = logging.getLogger("ditango_amd")
    root.setLevel(getattr(logging, os.environ.get("LOG_LEVEL", "INFO").upper(), logging.INFO))
    handler = logging.StreamHandler(sys.stdout)
    handler.setFormatter(logging.Formatter(_FORMAT, datefmt="%m-%d %H:%M:%S"))
    root.addHandler(handler)
    log_dir = os.environ.get("LOG_DIR")
    if log_dir:
        os.makedirs(log_dir, exist_ok=True)
        fh = logging.FileHandler(os.path.join(log_dir, f"process.{os.getpid()}.log"))
        fh.setFormatter(logging.Formatter(_FORMAT, datefmt="%m-%d %H:%M:%S"))
        root.addHandler(fh)
    root.propagate = False
    _configured = True


def init_logger(name: str) -> logging.Logger:
    _configure_root()
    if not name.startswith("ditango_amd"):
        name = "ditango_amd." + name
    return logging.getLogger(name)
