"""Build libditango_hip.so (gfx950) in-tree with hipcc.

``python -m ditango_amd.build`` compiles every translation unit under
``ditango_amd/csrc`` and links ``ditango_amd/lib/libditango_hip.so`` (the drop-in
library) and ``ditango_amd/lib/libditango_probes.so`` (the benchmark's measurement
aids, a library of its own that only ``bench.py`` loads).  hipcc
cross-compiles for gfx950 without a GPU.  Packed-FP32 instruction selection is
switched off for all device code (``-target-feature -packed-fp32-ops``).
"""
from __future__ import annotations

import json
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
LIB_DIR = PKG / "lib"
LIB_PATH = LIB_DIR / "libditango_hip.so"
PROBES_PATH = LIB_DIR / "libditango_probes.so"
DEMO_PATH = LIB_DIR / "dt_capi_demo"
RESOURCES_PATH = LIB_DIR / "kernel_resources.json"   # per-kernel registers / scratch / occupancy of the last build
SOURCES = ["attn_fwd.hip", "attn_f32.hip", "state_ops.hip", "producer.hip", "capi.hip"]
PROBE_SOURCES = ["probes.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    f"-I{ROOT / 'include'}", f"-I{CSRC}",
]


def _run(cmd):
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(map(str, cmd)) + "\n" + res.stdout + res.stderr)
    return res


def parse_resource_remarks(text: str) -> dict:
    """``{kernel symbol: {"VGPRs": n, "ScratchSize [bytes/lane]": n, ...}}`` from the compiler's
    ``-Rpass-analysis=kernel-resource-usage`` remarks."""
    out, cur = {}, None
    for line in text.splitlines():
        m = re.search(r"remark:\s+Function Name: (\S+)", line)
        if m:
            cur = out.setdefault(m.group(1), {})
            continue
        m = re.search(r"remark:\s+([A-Za-z][^:]*): (-?\d+)", line)
        if m and cur is not None:
            cur[m.group(1).strip()] = int(m.group(2))
    return out


def build_lib(verbose: bool = False, extra_flags=()) -> Path:
    """Compile and link the library unconditionally; returns its path."""
    LIB_DIR.mkdir(exist_ok=True)
    objs = []

    resources = {}

    def compile_one(src):
        obj = LIB_DIR / (Path(src).stem + ".o")
        # the resource remarks (registers, scratch, occupancy per kernel) come with the compilation at no cost
        cmd = [HIPCC, *COMMON, *extra_flags, "-Rpass-analysis=kernel-resource-usage", "-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        resources[src] = parse_resource_remarks(_run(cmd).stderr)
        return obj

    with ThreadPoolExecutor(max_workers=6) as ex:
        all_objs = list(ex.map(compile_one, SOURCES + PROBE_SOURCES))
    objs, probe_objs = all_objs[:len(SOURCES)], all_objs[len(SOURCES):]
    # a version script keeps everything but the C entry points out of the dynamic symbol table
    for out, members, exports in ((LIB_PATH, objs, "exports_hip.map"), (PROBES_PATH, probe_objs, "exports_probes.map")):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", f"-Wl,--version-script={CSRC / exports}",
               *map(str, members), "-o", str(out)]
        if verbose:
            print(" ".join(cmd), flush=True)
        _run(cmd)
    RESOURCES_PATH.write_text(json.dumps(resources, indent=1, sort_keys=True) + "\n")
    # a host program that uses nothing but the C header and the HIP runtime (tests/test_capi_demo_gpu.py runs it)
    cmd = [HIPCC, "-O2", "-std=c++17", "-Wno-unused-result", f"-I{ROOT / 'include'}", str(CSRC / "capi_demo.cpp"),
           f"-L{LIB_DIR}", "-lditango_hip", "-Wl,-rpath,$ORIGIN", "-o", str(DEMO_PATH)]
    if verbose:
        print(" ".join(cmd), flush=True)
    _run(cmd)
    return LIB_PATH


if __name__ == "__main__":
    path = build_lib(verbose=True)
    print(f"built {path}")
    sys.exit(0)
