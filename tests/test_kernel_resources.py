"""What the built library says about its own kernels (the AMDGPU metadata notes of the gfx950 code objects inside
libcomp_inference_hip.so): the register budgets the kernels' occupancy rests on, and the scratch (spill) bytes of the
kernels that have any.  The kernels are bound by wavefronts in flight, so a kernel that grows past its budget loses a
quarter or a third of its wavefronts per CU without a test result changing; this is where that shows without a GPU.

gfx950 has 512 VGPRs per SIMD lane: a workgroup of 1024 threads (four wavefronts per SIMD, the sixteen-wavefront
kernels) needs every wavefront within 128, one of 768 threads (three per SIMD) within 168, one of 512 within 256."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "comp_inference_amd", "libcomp_inference_hip.so")
OBJDUMP, READELF = "/opt/rocm/llvm/bin/llvm-objdump", "/opt/rocm/llvm/bin/llvm-readelf"

pytestmark = pytest.mark.skipif(not (os.path.exists(OBJDUMP) and os.path.exists(READELF) and os.path.exists(LIB)),
                                reason="needs the built library and the ROCm LLVM tools")

VGPR_BUDGET = {1024: 128, 768: 168, 512: 256, 256: 256, 64: 256}
# bytes of scratch per lane a kernel may use (every other kernel: none).  These are the figures of the build the
# measurements were taken on; more means new spills around the hand-scheduled loops.
SCRATCH_ALLOWED = {
    "fused_linear32_seg_kernel<1, false>": 16, "fused_linear32_seg_kernel<1, true>": 80,
    "fused_linear32_seg_kernel<2, false>": 80, "fused_linear32_seg_kernel<2, true>": 188,
    "fused_linear32_resident_kernel<1>": 100, "fused_linear32_resident_kernel<2>": 212, "trans32_kernel<4>": 44,
}
# kernels whose launch shape the host code relies on (threads per workgroup)
WORKGROUP = {"decode_tiled32_seg_kernel": 1024, "fused_linear32_seg_kernel": 1024, "embed_gather32_seg_kernel": 1024,
             "trans32_seg_kernel": 1024, "decode_tiled32_persist_kernel": 768, "fused_linear32_resident_kernel": 768,
             "embed_gather32_kernel": 768, "trans32_kernel": 768, "fused_linear32_kernel": 512, "fused_linear32_wide_kernel": 512}


@pytest.fixture(scope="module")
def kernels(tmp_path_factory):
    d = tmp_path_factory.mktemp("code_objects")
    shutil.copy(LIB, d / "lib.so")
    subprocess.run([OBJDUMP, "--offloading", "lib.so"], cwd=d, check=True, capture_output=True)  # writes lib.so.N.<target>
    out = {}
    for f in sorted(os.listdir(d)):
        if "gfx950" not in f:
            continue
        notes = subprocess.run([READELF, "--notes", str(d / f)], check=True, capture_output=True, text=True).stdout
        for block in notes.split("- .agpr_count:")[1:]:
            fields = dict(re.findall(r"\.(\w+):\s+(\S+)", ".agpr_count:" + block))
            name = subprocess.run(["c++filt", fields["name"]], capture_output=True, text=True).stdout.strip()
            out[name] = {k: int(fields[k]) for k in ("agpr_count", "vgpr_count", "sgpr_count", "private_segment_fixed_size",
                                                     "group_segment_fixed_size", "max_flat_workgroup_size")}
    assert len(out) >= 50, f"only {len(out)} kernels found: the notes were not understood"
    return out


def _short(name: str) -> str:
    return re.sub(r"^void ", "", name).replace("ci::", "").split("(")[0]


def test_register_budgets_hold_the_occupancy_the_kernels_are_built_for(kernels):
    for name, k in kernels.items():
        budget = VGPR_BUDGET[k["max_flat_workgroup_size"]]
        assert k["vgpr_count"] + k["agpr_count"] <= budget, \
            f"{_short(name)}: {k['vgpr_count']} + {k['agpr_count']} registers, {k['max_flat_workgroup_size']} threads allow {budget}"


def test_launch_shapes(kernels):
    seen = set()
    for name, k in kernels.items():
        for prefix, threads in WORKGROUP.items():
            if _short(name).split("<")[0] == prefix:
                assert k["max_flat_workgroup_size"] == threads, (name, k["max_flat_workgroup_size"])
                seen.add(prefix)
    assert seen == set(WORKGROUP), set(WORKGROUP) - seen


def test_scratch_use_has_not_grown(kernels):
    for name, k in kernels.items():
        allowed = SCRATCH_ALLOWED.get(_short(name), 0)
        assert k["private_segment_fixed_size"] <= allowed, \
            f"{_short(name)}: {k['private_segment_fixed_size']} bytes of scratch per lane, {allowed} before"


def test_static_lds_of_the_one_thread_per_stream_kernels(kernels):
    """Their slot table is a static array of 32 KB; the resident kernels ask for their LDS at launch (none static)."""
    for name, k in kernels.items():
        if "generic_kernel" in name or "checkpoints_kernel" in name or "decode_flat_kernel" in name or "decode_dense_kernel" in name:
            assert k["group_segment_fixed_size"] == 32768, (name, k["group_segment_fixed_size"])
        if any(p in name for p in ("_seg_kernel", "_persist_kernel", "_resident_kernel", "embed_gather32", "trans32_kernel")):
            assert k["group_segment_fixed_size"] == 0, (name, k["group_segment_fixed_size"])
