"""Per-kernel resource budget of the built code objects (registers, scratch, occupancy), from the compiler's
own resource remarks that ``ditango_amd.build`` records beside the library.  No GPU needed.

The attention kernel's arguments are a 3.6 KB struct.  A build in which the optimiser keeps a private copy of it
computes the same results -- every functional test passes -- but each lane copies the struct into scratch memory
before it starts, which multiplies the run time of a short launch.  Nothing but the scratch size shows it, so the
budget is pinned here."""
import json

import pytest


@pytest.fixture(scope="module")
def resources():
    from ditango_amd import build
    if not build.RESOURCES_PATH.exists() or not build.LIB_PATH.exists():
        build.build_lib()
    flat = {}
    for per_file in json.loads(build.RESOURCES_PATH.read_text()).values():
        flat.update(per_file)
    return flat


def _kernels(resources, fragment):
    found = {k: v for k, v in resources.items() if fragment in k}
    assert found, f"no kernel named like {fragment} in the build record"
    return found


def test_attention_kernel_keeps_its_arguments_out_of_scratch(resources):
    for name, r in _kernels(resources, "attn_fwd_kernel").items():
        d128 = "ILi128E" in name
        # a handful of spilled registers in the rare tile-redo branch at D = 64 is the budget; a private copy of the
        # argument struct would show up as thousands of bytes per lane
        assert r["ScratchSize [bytes/lane]"] <= (0 if d128 else 32), (name, r)
        assert r["VGPRs Spill"] <= (0 if d128 else 4), (name, r)
        # one workgroup of 8 wavefronts per CU at D = 128, two at D = 64
        assert r["Occupancy [waves/SIMD]"] == (2 if d128 else 4), (name, r)
        assert r["VGPRs"] <= (256 if d128 else 128), (name, r)


def test_streaming_kernels_use_no_scratch(resources):
    for fragment in ("merge_states_kernel", "flat_copy_kernel", "state_copy_kernel", "state_copy_units_kernel",
                     "rel_l1_sums_kernel", "qk_norm_rope_kernel", "attn_tail_fold_kernel", "build_schedule_kernel",
                     "zero_rows_from_kernel"):
        for name, r in _kernels(resources, fragment).items():
            assert r["ScratchSize [bytes/lane]"] == 0 and r["VGPRs Spill"] == 0, (name, r)


def test_remark_parser_reads_the_compilers_format():
    from ditango_amd.build import parse_resource_remarks
    text = ("x.hip:222:1: remark: Function Name: _ZN2dt3fooEv [-Rpass-analysis=kernel-resource-usage]\n"
            "x.hip:222:1: remark:     VGPRs: 128 [-Rpass-analysis=kernel-resource-usage]\n"
            "x.hip:222:1: remark:     ScratchSize [bytes/lane]: 20 [-Rpass-analysis=kernel-resource-usage]\n"
            "x.hip:222:1: remark:     Occupancy [waves/SIMD]: 4 [-Rpass-analysis=kernel-resource-usage]\n"
            "x.hip:900:1: remark: Function Name: _ZN2dt3barEv [-Rpass-analysis=kernel-resource-usage]\n"
            "x.hip:900:1: remark:     VGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]\n")
    got = parse_resource_remarks(text)
    assert got == {"_ZN2dt3fooEv": {"VGPRs": 128, "ScratchSize [bytes/lane]": 20, "Occupancy [waves/SIMD]": 4},
                   "_ZN2dt3barEv": {"VGPRs Spill": 0}}
