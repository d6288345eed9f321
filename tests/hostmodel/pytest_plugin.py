"""pytest plugin that runs tests written for the GPU on the host model instead:

    python -m pytest tests/test_gpu_runtime.py -m gpu -p tests.hostmodel.pytest_plugin

Every test runs inside tests/hostmodel/backend.python_api_on_hostmodel (the package's operators on CPU tensors, the
library being the host-model build), and ends with a check that the model reported nothing.  Tests that cannot mean
anything there are skipped with the reason: those that check that CPU tensors are refused, those that talk to
torch.cuda themselves, and those whose shapes would take the CPU model minutes."""
from __future__ import annotations

import pytest

NOT_APPLICABLE = {
    # the point of these is that a tensor which is not on the GPU is refused
    "test_python_layer_raises_runtime_error": "checks that CPU tensors are refused",
    "test_plain_weight_contraction_rejects_other_tilings": "checks that CPU tensors are refused",
    "test_dense_matmul_helper": "checks that CPU tensors are refused",
    "test_ops_refuse_cpu_tensors": "checks that CPU tensors are refused",
    # a module moved with .cuda() gets new tensors on a GPU and keeps its own here
    "test_rans_linear_prepares_once_and_follows_its_buffers": "asserts that .cuda() makes new tensors",
}
TOO_SLOW = ("test_gpu_full_size", "test_gpu_model", "test_gpu_random_sweep", "test_gpu_reference_sweep")
# single cases, by node id
CASES = {
    "2048-32800": "a 67 M-symbol weight: minutes on the CPU model (the resident kernel it selects runs in test_hostmodel_kernels.py)",
    "test_fused_kernels_above_64_rows[1300-80-1024-70]": "its last line asserts that hipBLASLt sums in another order than the "
                                                          "fused kernel; torch's CPU matmul happens to round this case the same way",
}


def pytest_collection_modifyitems(config, items):
    for item in items:
        name = item.originalname if hasattr(item, "originalname") else item.name
        if name in NOT_APPLICABLE:
            item.add_marker(pytest.mark.skip(reason="host model: " + NOT_APPLICABLE[name]))
        elif any(s in str(item.fspath) for s in TOO_SLOW):
            item.add_marker(pytest.mark.skip(reason="host model: shapes that take the CPU model minutes"))
        else:
            for piece, why in CASES.items():
                if piece in item.nodeid:
                    item.add_marker(pytest.mark.skip(reason="host model: " + why))


@pytest.fixture(autouse=True)
def _on_the_host_model():
    from tests.hostmodel.backend import python_api_on_hostmodel

    with python_api_on_hostmodel():
        yield
