"""The library's kernels compiled with the compiler's undefined-behaviour checks (tests/hostmodel/build.py,
`undefined=True`: array bounds, shift amounts, alignment of every typed access, null, signed overflow, pointer
arithmetic), run on the host model: a check that fires is a violation with the source position.  Code that is undefined
in C++ may compile to something else for the GPU than for the CPU model, so this is one more thing the model's results
rest on.  tests/test_hostmodel_selfcheck.py shows the checks firing on made-up kernels.

Every case of tests/test_hostmodel_kernels.py again, and a quarter of the random sweep (damaged contents included).  One
kind is let through, in sim.cpp: an offset added to a null pointer that is never read (`a.ckpt + ...` for a weight
without checkpoints, `a.man_tiled + ...` for a plain-weight run)."""
import os
import subprocess
import sys

import pytest

from tests.hostmodel import build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _lib():
    lib = build.build(undefined=True)
    build.build()  # (the children find both libraries up to date)
    return lib


def test_every_kernel_case_with_undefined_behaviour_checked():
    cmd = [sys.executable, "-m", "pytest", "tests/test_hostmodel_kernels.py", "-q", "-x", "-p", "no:cacheprovider", "-n", "6"]
    p = subprocess.run(cmd, cwd=ROOT, env=dict(os.environ, CI_HOSTMODEL_LIB=_lib()), capture_output=True, text=True, timeout=1500)
    assert p.returncode == 0 and " passed" in p.stdout and "failed" not in p.stdout, p.stdout[-6000:] + p.stderr[-2000:]


@pytest.mark.parametrize("family", ["decode", "fused_linear", "fused_gather", "lm_head", "other_layouts_and_encoders",
                                    "hand_scheduled_paths", "corrupted_contents"])
def test_random_cases_with_undefined_behaviour_checked(family, monkeypatch):
    from tests import test_hostmodel_sweep as sweep
    from tests.hostmodel.model import fork_all

    monkeypatch.setenv("CI_HOSTMODEL_LIB", _lib())
    fork_all(getattr(sweep, f"_blocks_of_test_{family}_sweep"), range(3))
