"""The built library loads and exports every function include/ditango_hip.h declares
(no compute calls: this runs without a GPU)."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "ditango_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dt_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared()
    for must in ("dt_attn_chunk_fwd", "dt_attn_jobs_fwd", "dt_attn_sched_fwd", "dt_merge_states", "dt_cache_store",
                 "dt_cache_load", "dt_build_schedule", "dt_build_schedule_table", "dt_rel_l1_sums", "dt_version",
                 "dt_last_error"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from ditango_amd import _hip
    if not _hip.LIB_PATH.exists():
        from ditango_amd.build import build_lib
        build_lib()
    lib = _hip.load_library()
    for name in _declared():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert set(_declared()) == set(_hip.EXPORTED_SYMBOLS)
    assert lib.dt_version() >= 100
    assert isinstance(lib.dt_last_error(), bytes)


def test_dynamic_symbol_table_holds_the_c_abi_and_nothing_else():
    """``nm -D``: the defined dynamic symbols of the drop-in library are exactly the header's functions (no C++
    internals, no kernel stubs, no measurement aids), and those of the probes library exactly ditango_probes.h's."""
    import shutil
    import subprocess
    from ditango_amd import _hip
    if shutil.which("nm") is None:
        pytest.skip("no nm")
    if not _hip.LIB_PATH.exists():
        from ditango_amd.build import build_lib
        build_lib()

    def defined(path):
        out = subprocess.run(["nm", "-D", "--defined-only", str(path)], capture_output=True, text=True, check=True).stdout
        return sorted(line.split()[-1] for line in out.splitlines() if line.split()[-2] in ("T", "t", "D", "B", "W"))

    assert defined(_hip.LIB_PATH) == _declared()
    assert not any("probe" in n for n in _declared())
    import bench_probes
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "ditango_probes.h")).read(), flags=re.S)
    probe_names = sorted(set(re.findall(r"\b(dtp_[a-z0-9_]+)\s*\(", text)))
    assert defined(bench_probes.PROBES_PATH) == probe_names == sorted(bench_probes.EXPORTED_SYMBOLS)
    lib = bench_probes.load_library()
    assert lib.dtp_mfma_probe(0, 4, None, None) == -1 and b"mfma probe" in lib.dtp_last_error()     # refused on the host


def test_every_entry_point_names_what_it_replaces():
    """Each declaration's comment cites the reference call site it stands in for (file.py:line) or says that
    the reference has no counterpart."""
    text = open(os.path.join(ROOT, "include", "ditango_hip.h")).read()
    body = text[text.index("int dt_version"):]
    blocks = re.findall(r"/\*(.*?)\*/(.*?)(?=/\*|#ifdef __cplusplus)", body, flags=re.S)
    seen = set()
    for comment, decls in blocks:
        names = re.findall(r"\b(dt_[a-z0-9_]+)\s*\(", decls)
        if not names:
            continue
        cites = re.search(r"[a-z_/]+\.py:\d+", comment) or "No counterpart in the reference" in comment \
            or "no counterpart in the reference" in comment
        assert cites, f"{names}: the comment names neither a reference call site nor the absence of one"
        seen.update(names)
    assert seen | {"dt_version", "dt_last_error"} == set(_declared())


def test_missing_library_fails_loudly(tmp_path):
    from ditango_amd import _hip
    with pytest.raises(_hip.DitangoHipError):
        _hip.load_library(tmp_path / "nope.so")


def test_argument_errors_are_reported_without_a_gpu():
    """Validation happens on the host before any launch."""
    from ditango_amd import _hip
    lib = _hip.load_library()
    rc = lib.dt_merge_states(0, None, None, None, None, None, 0, None, 0, 1, 1, 1, 128, None)
    assert rc == -1 and b"need 1.." in lib.dt_last_error()
    rc = lib.dt_attn_chunk_fwd(None, None, None, None, None, 1, 1, 1, 1, 96, 0, 0, 0, 0, 0, 0, 0.0, None)
    assert rc == -2 and b"head dim" in lib.dt_last_error()
    rc = lib.dt_build_schedule(None, 1, 1, 1, 0, 0, -1, None, None, None, None)
    assert rc == -1


def test_header_is_plain_c_and_links_from_c(tmp_path):
    """A C translation unit (gcc -std=c99 -pedantic) includes the header, takes the address of every
    declared function and links against the built library: the boundary has no C++ or torch types."""
    import shutil
    import subprocess
    from ditango_amd import _hip
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    if not _hip.LIB_PATH.exists():
        from ditango_amd.build import build_lib
        build_lib()
    names = _declared()
    src = tmp_path / "use.c"
    src.write_text('#include "ditango_hip.h"\n#include <stdio.h>\n'
                   "int main(void) {\n  void* p[] = {" + ", ".join(f"(void*){n}" for n in names) + "};\n"
                   "  int rc = dt_merge_states(0, 0, 0, 0, 0, 0, DT_BF16, 0, DT_LSE_BHS, 1, 1, 1, 128, 0);\n"
                   '  printf("%d %d %d %s\\n", dt_version(), (int)(sizeof(p) / sizeof(p[0])), rc, dt_last_error());\n'
                   "  return rc == DT_ERR_INVALID ? 0 : 1;\n}\n")
    exe = tmp_path / "use"
    libdir = str(_hip.LIB_PATH.parent)
    # -pedantic flags the function-pointer casts only; everything else must be clean
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe),
                        "-L", libdir, "-lditango_hip", f"-Wl,-rpath,{libdir}"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    ver, n, rc, *msg = r.stdout.split()
    assert int(ver) >= 100 and int(n) == len(names) and int(rc) == -1 and msg
