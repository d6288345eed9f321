"""Pins the oracle's plane split/merge, frequency table and decoder tables against what the
mathematics fixes, and the package's host functions against the oracle."""
import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_weight_kn, zipf_bytes


def test_split_merge_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    e, m = oracle.split_bf16(bits)
    # closed form, written on the bit layout s eeeeeeee mmmmmmm
    assert np.array_equal(e, ((bits >> 7) & 0xFF).astype(np.uint8))
    assert np.array_equal(m, (((bits >> 15) << 7) | (bits & 0x7F)).astype(np.uint8))
    assert np.array_equal(oracle.merge_bf16(e, m), bits)
    # every (exponent, sign|mantissa) pair is hit exactly once: the split is a bijection
    assert len(set(zip(e.tolist(), m.tolist()))) == 65536


def test_split_known_values(oracle):
    vals = torch.tensor([1.0, -1.0, 0.5, -0.0, 3.140625, float("inf")], dtype=torch.bfloat16)
    e, m = oracle.split_bf16(bf16_bits(vals))
    assert e.tolist() == [127, 127, 126, 0, 128, 255]
    assert m.tolist() == [0, 0x80, 0, 0x80, 0x49, 0]


def test_host_split_merge_matches_oracle(oracle):
    from comp_inference_amd import extract_exp_and_mantissa, reconstruct_from_exp_and_mantissa

    bits = np.arange(65536, dtype=np.uint16)
    t = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16)
    e, m = extract_exp_and_mantissa(t)
    eo, mo = oracle.split_bf16(bits)
    assert np.array_equal(e.numpy(), eo) and np.array_equal(m.numpy(), mo)
    back = reconstruct_from_exp_and_mantissa(e, m)
    assert np.array_equal(bf16_bits(back), bits)
    with pytest.raises(ValueError):
        extract_exp_and_mantissa(torch.zeros(4, dtype=torch.float16))


def _exact_floor_lut(data):
    """The table in exact integer arithmetic (no floating point)."""
    counts = np.bincount(data.reshape(-1), minlength=256).astype(object)
    total = int(counts.sum())
    f = [max(1, (int(c) * 4096) // total) for c in counts]
    diff = 4096 - sum(f)
    if diff > 0:
        f[f.index(max(f))] += diff
    while diff < 0:
        f[f.index(max(f))] -= 1
        diff += 1
    cdf = [0] * 256
    for i in range(1, 256):
        cdf[i] = cdf[i - 1] + f[i - 1]
    return np.array(f, np.uint16), np.array(cdf, np.uint16)


@pytest.mark.parametrize("case", ["weights", "zipf", "uniform", "single", "two", "ties"])
def test_lut_invariants_and_exact_floor(oracle, case):
    if case == "weights":
        data = oracle.split_bf16(bf16_bits(make_weight_kn(256, 512, 0)))[0]
    elif case == "zipf":
        data = zipf_bytes(100000, 2.0, 1)
    elif case == "uniform":
        data = np.arange(256, dtype=np.uint8).repeat(37)
    elif case == "single":
        data = np.full(1000, 77, np.uint8)
    elif case == "two":
        data = np.array([3] * 999 + [200], np.uint8)
    else:  # several symbols share the maximum: the first one absorbs the correction
        data = np.array([10] * 500 + [20] * 500 + [30] * 500 + [40] * 17, np.uint8)
    f, c = oracle.get_lut(data)
    assert int(f.astype(np.int64).sum()) == 4096 and f.min() >= 1
    assert c[0] == 0 and np.array_equal(c[1:], np.cumsum(f.astype(np.int64))[:-1])
    fe, ce = _exact_floor_lut(data)
    assert np.array_equal(f, fe) and np.array_equal(c, ce)
    if case == "single":
        assert f[77] == 4096 - 255 and (np.delete(f, 77) == 1).all()
    if case == "uniform":
        assert (f == 16).all()
    if case == "ties":
        # floor gives 1349 for each of 10/20/30; 253 forced ones push the sum over 4096 and the
        # excess is taken one unit at a time from the current first maximum
        assert f[10] <= f[20] <= f[30] and f[30] - f[10] <= 1


def test_host_lut_matches_oracle(oracle):
    from comp_inference_amd import get_rans_lut

    for seed in range(4):
        data = zipf_bytes(20000 + seed, 1.0 + seed, seed)
        f, c = oracle.get_lut(data)
        ft, ct = get_rans_lut(torch.from_numpy(data))
        assert ft.dtype == torch.uint16 and ct.dtype == torch.uint16
        assert np.array_equal(ft.view(torch.int16).numpy().view(np.uint16), f)
        assert np.array_equal(ct.view(torch.int16).numpy().view(np.uint16), c)


def test_decoder_tables_are_inverse_cdf(oracle):
    f, c = oracle.get_lut(zipf_bytes(50000, 1.5, 3))
    tables, slot_map = oracle.build_tables(f, c)
    assert np.array_equal(tables & 0xFFFF, f.astype(np.uint32))
    assert np.array_equal(tables >> 16, c.astype(np.uint32))
    slots = np.arange(4096)
    s = slot_map[slots].astype(np.int64)
    assert ((c[s] <= slots) & (slots < c[s].astype(np.int64) + f[s])).all()
    assert np.array_equal(np.bincount(slot_map, minlength=256), f.astype(np.int64))


@pytest.mark.parametrize("K,N,th,tw", [(1024, 64, 1024, 32), (1300, 70, 512, 32), (96, 40, 32, 16), (33, 5, 16, 8)])
def test_interleave_index_formula_and_inverse(oracle, K, N, th, tw):
    from comp_inference_amd import interleave_mantissas, uninterleave_mantissas

    rng = np.random.default_rng(K)
    plane = rng.integers(1, 256, size=(K, N), dtype=np.uint8)
    tiled = oracle.interleave_plane(plane, th, tw)
    tiles_n = -(-N // tw)
    assert tiled.size == -(-K // th) * tiles_n * th * tw
    for _ in range(200):
        r, c = int(rng.integers(K)), int(rng.integers(N))
        idx = ((r // th) * tiles_n + c // tw) * th * tw + (r % th) * tw + c % tw
        assert tiled[idx] == plane[r, c]
    assert int((tiled != 0).sum()) == K * N  # everything else is zero padding
    assert np.array_equal(oracle.uninterleave_plane(tiled, K, N, th, tw), plane)
    # a truncated tail reads back as zeros
    cut = oracle.uninterleave_plane(tiled[: tiled.size // 2], K, N, th, tw)
    assert cut.shape == (K, N)
    # host functions agree with the oracle
    ht = interleave_mantissas(torch.from_numpy(plane), TILE_K=th, TILE_N=tw)
    assert np.array_equal(ht.numpy(), tiled)
    assert np.array_equal(uninterleave_mantissas(ht, K, N, TILE_K=th, TILE_N=tw).numpy(), plane)
    assert np.array_equal(uninterleave_mantissas(ht[: ht.numel() // 2], K, N, TILE_K=th, TILE_N=tw).numpy(), cut)


@pytest.mark.parametrize("K,N,th,tw", [(256, 128, 128, 64), (300, 70, 128, 64), (96, 40, 32, 16)])
def test_halves_first_layout_of_the_sign_mantissa_plane(K, N, th, tw):
    """interleave_mantissas_ilp2 (comp_inference.py:96-153): per tile the top half's rows, then the bottom half's --
    element (tile row tk, tile column tn, half h, row r of the half, column c) at
    ((((tk * tiles_n + tn) * 2 + h) * th/2 + r) * tw + c, stated here from the reference's stack/view."""
    from comp_inference_amd import interleave_mantissas_ilp2, uninterleave_mantissas_ilp2

    rng = np.random.default_rng(K + N)
    plane = rng.integers(1, 256, size=(K, N), dtype=np.uint8)
    tiled = interleave_mantissas_ilp2(torch.from_numpy(plane), TILE_K=th, TILE_N=tw).numpy()
    tiles_n, half = -(-N // tw), th // 2
    assert tiled.size == -(-K // th) * tiles_n * th * tw
    for _ in range(300):
        r, c = int(rng.integers(K)), int(rng.integers(N))
        tk, tn, h, rr = r // th, c // tw, (r % th) // half, (r % th) % half
        assert tiled[((((tk * tiles_n + tn) * 2 + h) * half + rr) * tw) + c % tw] == plane[r, c]
    assert int((tiled != 0).sum()) == K * N
    assert np.array_equal(uninterleave_mantissas_ilp2(torch.from_numpy(tiled), K, N, TILE_K=th, TILE_N=tw).numpy(), plane)
    # the reference's defaults are 128 x 64
    assert np.array_equal(interleave_mantissas_ilp2(torch.from_numpy(plane)).numpy(),
                          interleave_mantissas_ilp2(torch.from_numpy(plane), 128, 64).numpy())
