"""Property tests of the CPU oracle over the parameter space the fixed cases sample: any shape,
any legal tile, any symbol distribution -- every layout round-trips, the two independent decoders
agree, and the packed layout keeps its invariants."""
import numpy as np
from hypothesis import given, settings, strategies as st

import pyref

L = 1 << 16


@st.composite
def planes(draw):
    th = draw(st.sampled_from([16, 32, 48, 64, 128]))
    tw = draw(st.sampled_from([1, 2, 8, 16, 32, 40]))
    K = draw(st.integers(1, 3 * th))
    N = draw(st.integers(1, 3 * tw))
    kind = draw(st.sampled_from(["uniform", "skewed", "two", "constant", "sparse_tail"]))
    seed = draw(st.integers(0, 2 ** 31 - 1))
    rng = np.random.default_rng(seed)
    if kind == "uniform":
        sym = rng.integers(0, 256, (K, N))
    elif kind == "skewed":
        p = 1.0 / np.arange(1, 257) ** draw(st.sampled_from([1.0, 2.0, 4.0]))
        sym = rng.choice(256, (K, N), p=p / p.sum())
    elif kind == "two":
        sym = rng.choice([draw(st.integers(0, 255)), draw(st.integers(0, 255))], (K, N))
    elif kind == "constant":
        sym = np.full((K, N), draw(st.integers(0, 255)))
    else:  # one dominant symbol, a few rare ones: long runs without a byte, then two bytes at once
        sym = np.where(rng.random((K, N)) < 0.98, 120, rng.integers(0, 256, (K, N)))
    return sym.astype(np.uint8), th, tw


def _encode(fn, *args):
    """The encoders refuse a stream that outgrows the reference's per-stream capacity (1.25 x the mean
    stream length + 64 bytes, src/cuda/rans_host.cuh:470-471), which ragged planes of poorly compressible
    symbols can do: such a case has nothing to round-trip."""
    try:
        return fn(*args)
    except RuntimeError as e:
        assert "capacity" in str(e)
        return None


@settings(max_examples=250, deadline=None, derandomize=True)
@given(planes())
def test_every_layout_round_trips(oracle, case):
    sym, th, tw = case
    K, N = sym.shape
    f, c = oracle.get_lut(sym)
    assert int(f.astype(np.int64).sum()) == 4096 and int(f.min()) >= 1

    enc = _encode(oracle.encode_tiled_ilp2, sym, f, c, th, tw)
    den = _encode(oracle.encode_tiled_dense, sym, f, c, th, tw)
    flat = _encode(oracle.encode_flat, sym, f, c, 512)
    if enc is None or den is None or flat is None:
        return
    spt = 2 * tw
    assert (enc.states >= L).all() and (enc.states < (1 << 24)).all()
    lens = enc.tile_max_lens.astype(np.int64) * spt
    assert np.array_equal(enc.tile_offsets.astype(np.int64), np.concatenate(([0], np.cumsum(lens)[:-1])))
    assert enc.stream.size == int(lens.sum())
    dec, end, left = oracle.decode_tiled_ilp2(enc.stream, enc.states, enc.tables, enc.slot_map, enc.tile_offsets,
                                              enc.tile_max_lens, K, N, th, tw, want_end=True)
    assert np.array_equal(dec, sym)
    assert (end == L).all()
    assert np.array_equal(left.astype(np.int64), np.repeat(enc.tile_max_lens, spt).astype(np.int64) - enc.sizes - 1)
    if K * N <= 2048:  # the numpy decoder is slow
        assert np.array_equal(pyref.decode_tiled(enc.stream, enc.states, enc.tables, enc.slot_map, enc.tile_offsets,
                                                 enc.tile_max_lens, K, N, th, tw), sym)

    assert np.array_equal(oracle.decode_tiled_dense(den.stream, den.states, den.tables, den.slot_map,
                                                    den.stream_offsets, den.sizes, K, N, th, tw), sym)
    assert den.stream.size == int(den.sizes.astype(np.int64).sum())

    # one stream per column in tile bodies: the dense layout's streams (same states, same lengths) packed like
    # the default layout's (bottom-aligned rows of tw bytes, offsets = scan of depth * tw)
    one = _encode(oracle.encode_tiled_one, sym, f, c, th, tw)
    if one is not None:
        assert np.array_equal(one.states, den.states) and np.array_equal(one.sizes, den.sizes)
        depth = one.tile_max_lens.astype(np.int64)
        assert np.array_equal(depth, one.sizes.reshape(-1, tw).max(1))
        assert np.array_equal(one.tile_offsets.astype(np.int64), np.concatenate(([0], np.cumsum(depth * tw)[:-1])))
        assert one.stream.size == int((depth * tw).sum())
        dec1, end1, left1 = oracle.decode_tiled_one(one.stream, one.states, one.tables, one.slot_map, one.tile_offsets,
                                                    one.tile_max_lens, K, N, th, tw, want_end=True)
        assert np.array_equal(dec1, sym) and (end1 == L).all()
        assert np.array_equal(left1.astype(np.int64), np.repeat(depth, tw) - one.sizes - 1)
        if K * N <= 2048:
            assert np.array_equal(pyref.decode_tiled(one.stream, one.states, one.tables, one.slot_map, one.tile_offsets,
                                                     one.tile_max_lens, K, N, th, tw, halves=1), sym)

    assert np.array_equal(oracle.decode_flat_segmented(flat.stream, flat.states, flat.sizes, flat.tables,
                                                       flat.slot_map, K, N), sym)


@settings(max_examples=150, deadline=None, derandomize=True)
@given(st.lists(st.integers(0, 255), min_size=1, max_size=96), st.integers(0, 2 ** 31 - 1))
def test_one_stream_equals_the_plain_integer_encoder(oracle, symbols, seed):
    """One column, one tile: the C encoder's state and bytes against the Python-integer encoder, with a
    table that need not match the data (any table with every frequency >= 1 codes any data)."""
    rng = np.random.default_rng(seed)
    sym = np.array(symbols, np.uint8).reshape(-1, 1)
    other = rng.integers(0, 256, 4096).astype(np.uint8)
    f, c = oracle.get_lut(np.concatenate([sym.reshape(-1), other]))
    n = sym.shape[0]
    th = -(-n // 16) * 16
    enc = oracle.encode_tiled_dense(sym, f, c, th, 1)
    x, out = pyref.encode_stream(sym[:, 0], f, c)
    assert int(enc.states[0]) == x and enc.stream.tolist() == out
