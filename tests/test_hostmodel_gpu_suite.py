"""The tests written for the GPU, run on the host model: `pytest -m gpu` of each test file with the plugin
tests/hostmodel/pytest_plugin.py, which puts every test inside tests/hostmodel/backend.python_api_on_hostmodel -- the
package's operators and modules on CPU tensors, the library underneath being the host-model build of the same
sources.  The same test code that runs on the MI355X therefore says, without one, that the Python layer and the
kernels of the current tree still produce what it asserts; this includes the files whose kernels have not run on a
GPU yet (tests/wip_*.py).  What the plugin skips, and why, is listed in it.  The files run side by side, each in a
process of its own."""
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# file -> tests that must at least have passed there (a guard against a run that silently collects nothing)
FILES = {"test_gpu_codec.py": 43, "test_gpu_linear.py": 65, "test_gpu_embedding.py": 18, "test_gpu_transposed.py": 21,
         "test_gpu_runtime.py": 10, "test_gpu_errors.py": 4, "test_golden.py": 1, "test_zz_no_alloc.py": 2,
         "test_gpu_zy_device_status.py": 1, "wip_one_stream.py": 15, "wip_transposed_seg.py": 10, "wip_linear_wide.py": 10,
         "wip_gather_seg.py": 8}


@pytest.fixture(scope="module")
def runs():
    from tests.hostmodel import build

    build.build()  # once, before the children would each try
    env = dict(os.environ, OMP_NUM_THREADS="2", PYTHONPATH=ROOT)
    procs = {f: subprocess.Popen([sys.executable, "-m", "pytest", os.path.join("tests", f), "-m", "gpu", "-q", "-p",
                                  "tests.hostmodel.pytest_plugin", "--timeout", "900", "-p", "no:cacheprovider"],
                                 cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
             for f in FILES}
    return {f: (p.communicate()[0], p.returncode) for f, p in procs.items()}


@pytest.mark.parametrize("name", list(FILES))
def test_gpu_tests_on_the_host_model(runs, name):
    out, rc = runs[name]
    assert rc == 0, out[-6000:]
    m = re.search(r"(\d+) passed", out)
    assert m and int(m.group(1)) >= FILES[name], out[-2000:]


def test_smoke_on_the_host_model():
    """__graft_entry__.smoke() -- encode, decode, fused linear against the oracle, on "cuda:0" -- on the host model."""
    code = ("import sys; sys.path.insert(0, %r); import __graft_entry__; "
            "from tests.hostmodel.backend import python_api_on_hostmodel\n"
            "with python_api_on_hostmodel():\n    __graft_entry__.smoke()\n") % ROOT
    p = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True)
    assert p.returncode == 0 and "smoke ok" in p.stdout, (p.stdout + p.stderr)[-3000:]
