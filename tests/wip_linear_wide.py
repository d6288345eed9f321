"""More than 64 rows of x through the fused linear with one decode per 128 or 256 rows
(`fused_wide_rows`): bit-identical to the kernel that decodes once per 64 rows, and within the reference's
tolerance of torch.matmul (tests/test_mat_mul.py:220).

Not collected by pytest until it has passed on the GPU (run it by naming the file)."""
import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_weight_kn, make_x

pytestmark = pytest.mark.gpu

ATOL = RTOL = 1e-2


def _t32(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int32))


@pytest.fixture
def always_fused():
    import comp_inference_amd.linear_hip as lh

    old = lh.DECODE_ONCE_ABOVE_ROWS
    lh.DECODE_ONCE_ABOVE_ROWS = None
    yield lh
    lh.DECODE_ONCE_ABOVE_ROWS = old
    lh.fused_wide_rows(False)


def _call(oracle, lh, w, x, th, bias=None):
    K, N = w.shape
    enc, man = oracle.compress_bf16(bf16_bits(w), th, 32)
    dev = "cuda"
    args = (torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
            torch.from_numpy(enc.slot_map).to(dev), (K, N), _t32(enc.tile_offsets).to(dev),
            _t32(enc.tile_max_lens).to(dev), th, 32, torch.from_numpy(man).to(dev))
    out = {}
    for wide in (False, True):
        lh.fused_wide_rows(wide)
        out[wide] = lh.fused_rans_linear(x.to(dev), *args, bias=None if bias is None else bias.to(dev))
    return out


@pytest.mark.parametrize("K,N,th,M", [
    (1024, 64, 1024, 65), (1024, 64, 1024, 128), (1024, 96, 1024, 129), (2048, 128, 1024, 200),
    (4096, 256, 1024, 256), (4096, 64, 1024, 257), (2048, 64, 512, 600),
    (700, 64, 1024, 100),     # a short tile row: guarded steps
    (1024, 50, 1024, 150),    # ragged columns
])
def test_wide_rows_are_bit_identical_and_close_to_matmul(oracle, always_fused, K, N, th, M):
    w = make_weight_kn(N, K, seed=K + M)
    x = make_x(M, K, seed=M)
    bias = make_x(1, N, seed=7).view(N)
    out = _call(oracle, always_fused, w, x, th, bias)
    assert out[True].shape == (M, N)
    assert torch.equal(out[True], out[False])
    want = torch.matmul(x.float(), w.float()) + bias.float()
    assert torch.allclose(out[True].float().cpu(), want, atol=ATOL, rtol=RTOL), (out[True].float().cpu() - want).abs().max()


def test_wide_rows_with_a_strided_x(oracle, always_fused):
    K, N, th, M = 2048, 64, 1024, 130
    w = make_weight_kn(N, K, seed=3)
    x = make_x(M, K + 64, seed=5)[:, :K]      # rows 64 elements apart from contiguous
    out = _call(oracle, always_fused, w, x, th)
    assert torch.equal(out[True], out[False])
    want = torch.matmul(x.float(), w.float())
    assert torch.allclose(out[True].float().cpu(), want, atol=ATOL, rtol=RTOL)
