"""GPU parity of the row-per-output (LM head) fused linear against torch.matmul on the
oracle-decoded weight, tolerance as the reference's own test (atol = rtol = 1e-2)."""
import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_weight_kn, make_x

pytestmark = pytest.mark.gpu
ATOL = RTOL = 1e-2


def _t32(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int32))


@pytest.mark.parametrize("V,H,th,tw,M", [
    (2048, 128, 1024, 32, 1), (1300, 96, 1024, 32, 1), (1300, 96, 1024, 32, 3), (2048, 64, 512, 32, 6),
    (700, 100, 256, 32, 2), (300, 48, 64, 16, 2), (512, 128, 128, 64, 1),
])
def test_transposed_linear(oracle, V, H, th, tw, M):
    from comp_inference_amd import fused_rans_linear_transposed_triton

    w = make_weight_kn(H, V, seed=V + H)  # [V, H]: rows are outputs
    enc, man = oracle.compress_bf16(bf16_bits(w), th, tw)
    x = make_x(M, H, seed=M)
    dev = "cuda"
    got = fused_rans_linear_transposed_triton(
        x.to(dev), torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
        torch.from_numpy(enc.slot_map).to(dev), (V, H), _t32(enc.tile_offsets).to(dev),
        _t32(enc.tile_max_lens).to(dev), th, tw, torch.from_numpy(man).to(dev), workspace=None)
    want = torch.matmul(x.float(), w.float().t())
    assert got.shape == (M, V) and got.dtype == torch.bfloat16
    assert torch.allclose(got.float().cpu(), want, atol=ATOL, rtol=RTOL), (got.float().cpu() - want).abs().max()
    again = fused_rans_linear_transposed_triton(
        x.to(dev), torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
        torch.from_numpy(enc.slot_map).to(dev), (V, H), _t32(enc.tile_offsets).to(dev),
        _t32(enc.tile_max_lens).to(dev), th, tw, torch.from_numpy(man).to(dev), workspace=None)
    assert torch.equal(got, again)  # fixed summation order


def test_transposed_linear_dense_layout(oracle):
    from comp_inference_amd import fused_rans_linear_transposed_triton_uncoalesced

    V, H, th, tw, M = 600, 64, 256, 32, 2
    w = make_weight_kn(H, V, seed=5)
    e, m = oracle.split_bf16(bf16_bits(w))
    f, c = oracle.get_lut(e)
    enc = oracle.encode_tiled_dense(e, f, c, th, tw)
    man = oracle.interleave_plane(m, th, tw)
    x = make_x(M, H, seed=6)
    dev = "cuda"
    got = fused_rans_linear_transposed_triton_uncoalesced(
        x.to(dev), torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
        torch.from_numpy(enc.slot_map).to(dev), (V, H), _t32(enc.stream_offsets).to(dev), _t32(enc.sizes).to(dev),
        th, tw, torch.from_numpy(man).to(dev), workspace=None)
    want = torch.matmul(x.float(), w.float().t())
    assert torch.allclose(got.float().cpu(), want, atol=ATOL, rtol=RTOL)
