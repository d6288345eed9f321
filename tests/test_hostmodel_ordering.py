"""The library's kernels under the ordering check of the host model (tests/hostmodel/build.py, `order=True`): the kernel
sources compiled with the compiler's thread-sanitizer instrumentation, every plain memory access reported to the model,
which keeps a vector clock per wavefront and reports two wavefronts that touch the same byte of the LDS (or two
workgroups the same byte of an array) with no barrier or release / acquire pair between them.  The plain model runs the
wavefronts one after the other, so a missing barrier changes nothing there; on the GPU it is a wrong result now and
then.  tests/test_hostmodel_selfcheck.py shows that the check fires on made-up kernels, tests/test_hostmodel_mutants.py
that it fires when a barrier or a release is taken out of the real ones.

Here: every case of tests/test_hostmodel_kernels.py again on that build (each case asserts that the model reported
nothing), and half of the random sweep's blocks of every family whose inputs an encoder wrote (about 2,000 cases)."""
import os
import subprocess
import sys

import pytest

from tests.hostmodel import build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# Cases in which unordered accesses are what the case is about, not a defect:
BY_DESIGN = [
    # the wait between wavefronts is forced to give up: the hand-over it guards is then unordered, which is why it is there
    "tests/test_hostmodel_kernels.py::test_the_bounded_wait_gives_up_and_says_so",
    # tile metadata that is noise: the decoder runs on noise as well and takes bytes from below its window, another
    # wavefront's (inside the LDS; the values are garbage either way)
    "tests/test_hostmodel_kernels.py::test_tile_metadata_that_points_past_the_stream_is_not_followed",
]


def _env():
    env = dict(os.environ)
    env["CI_HOSTMODEL_LIB"] = build.build(order=True)
    build.build()  # (the children find both libraries up to date)
    return env


def _kernels_the_host_code_can_launch():
    """Every kernel instance named in a launch of the library's sources."""
    import glob
    import re

    names = set()
    for path in glob.glob(os.path.join(ROOT, "comp_inference_amd", "csrc", "*.hip")):
        for m in re.finditer(r"hipLaunchKernelGGL\(\s*\(?\s*([a-z0-9_]+(?:<[^>]*>)?)", open(path).read()):
            names.add(m.group(1).replace(" ", ""))
    macro = "fused_linear32_seg_kernel<MB_,COLD_>"  # (instantiated for one and two groups of rows, with and without guarded path)
    assert macro in names
    names.remove(macro)
    names |= {f"fused_linear32_seg_kernel<{mb},{cold}>" for mb in (1, 2) for cold in ("true", "false")}
    return names


def test_every_kernel_case_with_ordering_checked(tmp_path):
    """... and, from the same run's log of launches: the cases reach every kernel instance the host code can launch."""
    cmd = [sys.executable, "-m", "pytest", "tests/test_hostmodel_kernels.py", "-q", "-x", "-p", "no:cacheprovider", "-n", "6"]
    for case in BY_DESIGN:
        cmd += ["--deselect", case]
    log = tmp_path / "launches.log"
    p = subprocess.run(cmd, cwd=ROOT, env=dict(_env(), CI_HOSTMODEL_LAUNCH_LOG=str(log)), capture_output=True, text=True, timeout=1500)
    assert p.returncode == 0, p.stdout[-6000:] + p.stderr[-2000:]
    assert " passed" in p.stdout and "failed" not in p.stdout, p.stdout[-2000:]
    launched = {line.strip().strip("()").replace(" ", "") for line in log.read_text().splitlines() if not line.startswith("st_")}
    can = _kernels_the_host_code_can_launch()
    assert len(can) > 50 and can - launched == set(), f"kernels no case of tests/test_hostmodel_kernels.py launches: {sorted(can - launched)}"


def test_the_forced_give_up_is_seen_as_what_it_is():
    """The one case whose hand-over is unordered on purpose is reported as such -- on the real kernel, by the flag
    protocol's own accesses."""
    cmd = [sys.executable, "-m", "pytest", BY_DESIGN[0], "-q", "-x", "-p", "no:cacheprovider"]
    p = subprocess.run(cmd, cwd=ROOT, env=_env(), capture_output=True, text=True, timeout=600)
    assert p.returncode != 0 and "ordering:" in p.stdout and "fused_linear32_seg_kernel" in p.stdout, p.stdout[-3000:]


@pytest.mark.parametrize("family", ["decode", "fused_linear", "fused_gather", "lm_head", "other_layouts_and_encoders",
                                    "hand_scheduled_paths"])
def test_random_cases_with_ordering_checked(family, monkeypatch):
    from tests import test_hostmodel_sweep as sweep
    from tests.hostmodel.model import fork_all

    monkeypatch.setenv("CI_HOSTMODEL_LIB", _env()["CI_HOSTMODEL_LIB"])
    fork_all(getattr(sweep, f"_blocks_of_test_{family}_sweep"), range(6))


def test_the_gpu_tests_of_the_operators_with_ordering_checked():
    """The tests written for the GPU (tests/test_hostmodel_gpu_suite.py runs them on the plain model), on this build:
    the operators' files, the runtime modules, the entry point without allocation and the four files whose kernels have
    not run on a GPU.  Their tensors are torch's, memory that is
    not the model's, so what is checked here is the LDS side; the arrays are checked in the cases above."""
    files = ["test_gpu_codec.py", "test_gpu_linear.py", "test_gpu_embedding.py", "test_gpu_transposed.py",
             "test_gpu_runtime.py", "test_zz_no_alloc.py", "test_golden.py",
             "wip_one_stream.py", "wip_transposed_seg.py", "wip_linear_wide.py", "wip_gather_seg.py"]
    env = dict(_env(), OMP_NUM_THREADS="2", PYTHONPATH=ROOT)
    procs = {f: subprocess.Popen([sys.executable, "-m", "pytest", os.path.join("tests", f), "-m", "gpu", "-q", "-p",
                                  "tests.hostmodel.pytest_plugin", "--timeout", "900", "-p", "no:cacheprovider"],
                                 cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
             for f in files}
    for f, p in procs.items():
        out = p.communicate()[0]
        assert p.returncode == 0 and " passed" in out, f + ":\n" + out[-6000:]
