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


@pytest.mark.parametrize("V,H,th,M", [
    (2048, 128, 1024, 1), (2048, 128, 1024, 4), (2048, 128, 1024, 6),
    (1300, 96, 1024, 1),    # short last tile row: the bottom half has fewer rows than the top half
    (1300, 96, 1024, 3),
    (2048, 64, 512, 2),
    (700, 100, 256, 2),     # ragged columns: guarded steps in both runs
])
def test_transposed_linear_bit_identical_to_plain_weight_contraction(oracle, V, H, th, M):
    """Fused kernel on the compressed [V, H] weight == the same products and reductions on the plain bf16
    weight, bit for bit (sharper than the tolerance against torch.matmul)."""
    from comp_inference_amd import fused_rans_linear_transposed_triton, plain_linear_transposed_same_order

    w = make_weight_kn(H, V, seed=V + H + 1)  # [V, H]
    enc, man = oracle.compress_bf16(bf16_bits(w), th, 32)
    x = make_x(M, H, seed=M + 20)
    dev = "cuda"
    got = fused_rans_linear_transposed_triton(
        x.to(dev), torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
        torch.from_numpy(enc.slot_map).to(dev), (V, H), _t32(enc.tile_offsets).to(dev),
        _t32(enc.tile_max_lens).to(dev), th, 32, torch.from_numpy(man).to(dev), workspace=None)
    same = plain_linear_transposed_same_order(x.to(dev), w.to(dev), tile_k=th, tile_n=32)
    assert torch.equal(got.view(torch.int16), same.view(torch.int16))
    want = torch.matmul(x.float(), w.float().t())
    assert torch.allclose(same.float().cpu(), want, atol=ATOL, rtol=RTOL)


def test_transposed_guarded_and_fast_tiles_sum_alike(oracle):
    """A tile's partial sums do not depend on the path it took: bodies too deep for the staging area
    (nearly incompressible exponents) take guarded steps, and still match the plain-weight contraction."""
    from comp_inference_amd import fused_rans_linear_transposed_triton, plain_linear_transposed_same_order

    V, H, th, M = 2048, 64, 1024, 2
    rng = np.random.default_rng(5)
    bits = rng.integers(0, 1 << 16, size=(V, H), dtype=np.uint16)
    bits = (bits & 0x807F) | (rng.integers(100, 140, size=(V, H)).astype(np.uint16) << 7)  # 40 exponents, finite
    w = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16)
    enc, man = oracle.compress_bf16(bits, th, 32)
    assert int(enc.tile_max_lens.max()) >= 254      # deeper than the largest lane stride
    x = make_x(M, H, seed=9)
    dev = "cuda"
    got = fused_rans_linear_transposed_triton(
        x.to(dev), torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
        torch.from_numpy(enc.slot_map).to(dev), (V, H), _t32(enc.tile_offsets).to(dev),
        _t32(enc.tile_max_lens).to(dev), th, 32, torch.from_numpy(man).to(dev), workspace=None)
    same = plain_linear_transposed_same_order(x.to(dev), w.to(dev), tile_k=th, tile_n=32)
    assert torch.equal(got.view(torch.int16), same.view(torch.int16))


@pytest.mark.parametrize("V,H,th,M", [(2048, 128, 1024, 6), (1300, 96, 1024, 9), (2048, 64, 512, 5)])
def test_transposed_fused_kernel_above_4_rows(oracle, always_fused, V, H, th, M):
    """With the decode-once policy off, more than 4 rows run the fused kernel in passes of 4."""
    from comp_inference_amd import fused_rans_linear_transposed_triton, plain_linear_transposed_same_order

    w = make_weight_kn(H, V, seed=V + M)
    enc, man = oracle.compress_bf16(bf16_bits(w), th, 32)
    x = make_x(M, H, seed=M + 40)
    dev = "cuda"
    got = fused_rans_linear_transposed_triton(
        x.to(dev), torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
        torch.from_numpy(enc.slot_map).to(dev), (V, H), _t32(enc.tile_offsets).to(dev),
        _t32(enc.tile_max_lens).to(dev), th, 32, torch.from_numpy(man).to(dev), workspace=None)
    want = torch.matmul(x.float(), w.float().t())
    assert torch.allclose(got.float().cpu(), want, atol=ATOL, rtol=RTOL)
    same = plain_linear_transposed_same_order(x.to(dev), w.to(dev), tile_k=th, tile_n=32)
    assert torch.equal(got.view(torch.int16), same.view(torch.int16))


def test_transposed_many_rows_decode_the_weight_once(oracle):
    """Above DECODE_ONCE_ABOVE_ROWS rows: torch.matmul on the weight decoded once, bit for bit."""
    from comp_inference_amd import fused_rans_linear_transposed_triton

    V, H, th, M = 1300, 96, 1024, 20
    w = make_weight_kn(H, V, seed=51)
    enc, man = oracle.compress_bf16(bf16_bits(w), th, 32)
    x = make_x(M, H, seed=52).cuda()
    dev = "cuda"
    got = fused_rans_linear_transposed_triton(
        x, torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
        torch.from_numpy(enc.slot_map).to(dev), (V, H), _t32(enc.tile_offsets).to(dev),
        _t32(enc.tile_max_lens).to(dev), th, 32, torch.from_numpy(man).to(dev), workspace=None)
    want = torch.matmul(x, w.cuda().t())
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_transposed_random_shapes(oracle, always_fused):
    """Twenty seeded random [V, H] weights (ragged, 1 to 9 rows of x, three tile heights) on the fused kernel:
    within tolerance of torch.matmul and bit-identical to the plain-weight contraction."""
    from comp_inference_amd import fused_rans_linear_transposed_triton, plain_linear_transposed_same_order

    rng = np.random.default_rng(55)
    dev = "cuda"
    for case in range(20):
        th = int(rng.choice([64, 256, 1024]))
        V = int(rng.integers(1, 3 * th + 1))
        H = int(rng.integers(8, 200))
        M = int(rng.integers(1, 10))
        w = make_weight_kn(H, V, seed=6000 + case)  # [V, H]
        enc, man = oracle.compress_bf16(bf16_bits(w), th, 32)
        x = make_x(M, H, seed=7000 + case)
        got = fused_rans_linear_transposed_triton(
            x.to(dev), torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
            torch.from_numpy(enc.slot_map).to(dev), (V, H), _t32(enc.tile_offsets).to(dev),
            _t32(enc.tile_max_lens).to(dev), th, 32, torch.from_numpy(man).to(dev), workspace=None)
        want = torch.matmul(x.float(), w.float().t())
        assert torch.allclose(got.float().cpu(), want, atol=ATOL, rtol=RTOL), (case, V, H, M, th)
        same = plain_linear_transposed_same_order(x.to(dev), w.to(dev), tile_k=th, tile_n=32)
        assert torch.equal(got.view(torch.int16), same.view(torch.int16)), (case, V, H, M, th)
