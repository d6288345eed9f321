"""Pins the oracle's coders: algebraic inverse of one step, state interval, exact end state,
information-theoretic size, closed forms, packed-layout invariants, an independent second
implementation, and round trips of every layout including ragged and empty cases."""
import math

import numpy as np
import pytest

import pyref
from helpers import bf16_bits, make_weight_kn, zipf_bytes

L, M = 1 << 16, 1 << 12


def _table(oracle, data):
    f, c = oracle.get_lut(data)
    return f, c


def test_decode_step_inverts_encode_step(oracle):
    """D(C(x, s)) = (x, s) for every symbol and a sweep of states: fixed by the algebra
    C = floor(x/f)*M + x mod f + c, slot = C mod M in [c, c+f)."""
    f, c = _table(oracle, zipf_bytes(30000, 1.3, 0))
    tables, slot_map = oracle.build_tables(f, c)
    xs = np.unique(np.concatenate([np.arange(L, L + 300), np.arange((1 << 24) - 300, 1 << 24),
                                   np.random.default_rng(0).integers(L, 1 << 24, 2000)])).astype(np.int64)
    for s in range(256):
        fs, cs = int(f[s]), int(c[s])
        xr = xs[xs < ((L >> 12) << 8) * fs]  # states the encoder can hold before coding s
        C = (xr // fs) * M + xr % fs + cs
        slot = C & (M - 1)
        assert (slot_map[slot] == s).all()
        assert np.array_equal(fs * (C >> 12) + slot - cs, xr)


def test_single_stream_matches_python_encoder_and_interval(oracle):
    rng = np.random.default_rng(1)
    sym = zipf_bytes(16 * 1, 1.2, 2).reshape(16, 1)
    for n in (16, 48, 512):
        sym = zipf_bytes(n, 1.2, n).reshape(n, 1)
        f, c = _table(oracle, sym)
        enc = oracle.encode_tiled_dense(sym, f, c, n, 1)  # one tile, one column, one stream
        x, out = pyref.encode_stream(sym[:, 0], f, c)
        assert enc.states[0] == x and enc.stream.tolist() == out
        assert L <= x < (1 << 24)


@pytest.mark.parametrize("K,N,th,tw", [(1024, 64, 1024, 32), (2048, 32, 1024, 32), (1300, 80, 1024, 32),
                                       (1000, 70, 512, 32), (96, 100, 32, 32), (256, 48, 64, 16), (48, 8, 16, 8)])
def test_tiled_roundtrip_end_state_and_layout(oracle, K, N, th, tw):
    sym = oracle.split_bf16(bf16_bits(make_weight_kn(N, K, K + N)))[0]
    f, c = _table(oracle, sym)
    enc = oracle.encode_tiled_ilp2(sym, f, c, th, tw)
    tiles_k, tiles_n, spt = -(-K // th), -(-N // tw), 2 * tw
    assert (enc.num_tiles_k, enc.num_tiles_n, enc.num_streams) == (tiles_k, tiles_n, tiles_k * tiles_n * spt)
    # state interval after encoding
    assert (enc.states >= L).all() and (enc.states < (1 << 24)).all()
    # packed layout: offsets are the running sum of max_len * 2tw, length matches, no gaps
    lens = enc.tile_max_lens.astype(np.int64) * spt
    assert np.array_equal(enc.tile_offsets.astype(np.int64), np.concatenate(([0], np.cumsum(lens)[:-1])))
    assert enc.stream.size == int(lens.sum())
    sizes = enc.sizes.reshape(-1, spt)
    assert np.array_equal(sizes.max(axis=1), enc.tile_max_lens)
    # every stream is bottom aligned under a zero prefix
    for t in (0, tiles_k * tiles_n - 1):
        body = enc.stream[enc.tile_offsets[t]: enc.tile_offsets[t] + lens[t]].reshape(-1, spt)
        for q in range(spt):
            pad = int(enc.tile_max_lens[t] - sizes[t, q])
            assert not body[:pad, q].any()
    # decode: exact symbols, every stream ends on state 2^16 with exactly its own bytes consumed
    dec, end, left = oracle.decode_tiled_ilp2(enc.stream, enc.states, enc.tables, enc.slot_map, enc.tile_offsets,
                                              enc.tile_max_lens, K, N, th, tw, want_end=True)
    assert np.array_equal(dec, sym)
    assert (end == L).all()
    pad_rows = np.repeat(enc.tile_max_lens, spt).astype(np.int64) - enc.sizes
    assert np.array_equal(left.astype(np.int64), pad_rows - 1)
    # streams of rows >= K or columns >= N are empty
    lane_col = (np.arange(enc.num_streams) // spt % tiles_n) * tw + np.arange(enc.num_streams) % tw
    assert (enc.sizes[lane_col >= N] == 0).all() and (enc.states[lane_col >= N] == L).all()


def test_second_implementation_agrees(oracle):
    K, N, th, tw = 80, 24, 32, 8
    sym = zipf_bytes(K * N, 1.1, 9).reshape(K, N)
    f, c = _table(oracle, sym)
    enc = oracle.encode_tiled_ilp2(sym, f, c, th, tw)
    got = pyref.decode_tiled(enc.stream, enc.states, enc.tables, enc.slot_map, enc.tile_offsets,
                             enc.tile_max_lens, K, N, th, tw)
    assert np.array_equal(got, sym)
    # and the encoder, stream by stream, against the plain-integer encoder
    spt, half, tiles_n = 2 * tw, th // 2, -(-N // tw)
    for sid in range(0, enc.num_streams, 5):
        t, q = divmod(sid, spt)
        tk, tn = divmod(t, tiles_n)
        col, r0 = tn * tw + q % tw, tk * th + (q // tw) * half
        rows = [r for r in range(r0, r0 + half) if r < K]
        if col >= N:
            continue
        x, out = pyref.encode_stream(sym[rows, col], f, c)
        assert enc.states[sid] == x and enc.sizes[sid] == len(out)
        pad = int(enc.tile_max_lens[t]) - len(out)
        body = enc.stream[enc.tile_offsets[t]:][: int(enc.tile_max_lens[t]) * spt].reshape(-1, spt)
        assert body[pad:, q].tolist() == out


def test_compressed_size_tracks_cross_entropy(oracle):
    """bytes*8 + log2(state/L) of a stream is the code length: sum of -log2(f/4096) up to the
    coder's sub-bit slack per renormalisation."""
    K, N = 1024, 64
    sym = oracle.split_bf16(bf16_bits(make_weight_kn(N, K, 5)))[0]
    f, c = _table(oracle, sym)
    enc = oracle.encode_tiled_ilp2(sym, f, c, 1024, 32)
    cost = -np.log2(f.astype(np.float64) / 4096.0)
    ideal_bits = cost[sym].sum()
    got_bits = enc.sizes.astype(np.float64).sum() * 8 + np.log2(enc.states.astype(np.float64) / L).sum()
    assert abs(got_bits - ideal_bits) / ideal_bits < 2e-3


def test_closed_form_power_of_two_frequencies(oracle):
    """A symbol of frequency 2^k costs exactly 12-k bits: n such symbols take
    floor(n*(12-k)/8) bytes (+-1 for the final partial byte kept in the state)."""
    n = 512
    freq = np.ones(256, np.uint16)
    freq[7] = 2048
    freq[9] = 4096 - 2048 - 254
    cdf = np.concatenate(([0], np.cumsum(freq.astype(np.int64))[:-1])).astype(np.uint16)
    sym = np.full((n, 1), 7, np.uint8)
    enc = oracle.encode_tiled_dense(sym, freq, cdf, n, 1)
    bits = enc.sizes[0] * 8 + math.log2(enc.states[0] / L)
    assert abs(bits - n * 1.0) < 1e-6 + 1.0
    assert abs(int(enc.sizes[0]) - n // 8) <= 1
    n = 128  # frequency 1: 12 bits each (kept short: such a stream is near the capacity limit)
    sym = np.full((n, 1), 3, np.uint8)
    enc = oracle.encode_tiled_dense(sym, freq, cdf, n, 1)
    assert abs(int(enc.sizes[0]) - n * 12 // 8) <= 2
    dec = oracle.decode_tiled_dense(enc.stream, enc.states, enc.tables, enc.slot_map, enc.stream_offsets,
                                    enc.sizes, n, 1, n, 1)
    assert (dec == 3).all()


@pytest.mark.parametrize("K,N,th,tw", [(1024, 64, 1024, 32), (700, 50, 256, 32), (100, 9, 64, 16)])
def test_dense_roundtrip(oracle, K, N, th, tw):
    sym = zipf_bytes(K * N, 1.5, 3).reshape(K, N)
    f, c = _table(oracle, sym)
    enc = oracle.encode_tiled_dense(sym, f, c, th, tw)
    assert np.array_equal(enc.stream_offsets.astype(np.int64),
                          np.concatenate(([0], np.cumsum(enc.sizes.astype(np.int64))[:-1])))
    assert enc.stream.size == int(enc.sizes.sum())
    dec, end, left = oracle.decode_tiled_dense(enc.stream, enc.states, enc.tables, enc.slot_map,
                                               enc.stream_offsets, enc.sizes, K, N, th, tw, want_end=True)
    assert np.array_equal(dec, sym) and (end == L).all() and (left == 0).all()


@pytest.mark.parametrize("K,N", [(300, 8), (512, 33), (1500, 16), (5000, 1)])
def test_flat_roundtrip_and_checkpoints(oracle, K, N):
    sym = zipf_bytes(K * N, 4.0, 11).reshape(K, N)
    f, c = _table(oracle, sym)
    enc = oracle.encode_flat(sym, f, c, 512)
    S = -(-K // 512) * N
    assert enc.num_streams == S and enc.stream.size == int(enc.sizes.max()) * S
    assert np.array_equal(oracle.decode_flat_segmented(enc.stream, enc.states, enc.sizes, enc.tables,
                                                       enc.slot_map, K, N), sym)
    # checkpoint 0 of every non-empty stream is the initial state with nothing written
    assert (enc.checkpoints[:S] == L).all()
    # the extension's own flat decoder agrees with [row, col] order only when one segment covers K
    strided = oracle.decode_flat_strided(enc.stream, enc.states, enc.sizes, enc.tables, enc.slot_map, K * N)
    assert np.array_equal(strided.reshape(K, N), sym) == (K <= 512)


def test_flat_stream_count_follows_min_block(oracle):
    assert oracle.flat_num_streams(1000, 4, 512) == 8
    assert oracle.flat_num_streams(1000, 4, 256) == 16
    sym = zipf_bytes(1000 * 4, 2.0, 1).reshape(1000, 4)
    f, c = _table(oracle, sym)
    enc = oracle.encode_flat(sym, f, c, 256)  # twice the streams, the extra ones stay empty
    assert (enc.sizes[8:] == 0).all() and (enc.states[8:] == L).all()


def test_capacity_overflow_is_reported(oracle):
    """Symbols that all cost 12 bits outgrow the reference's per-stream capacity
    (1.25 bytes per symbol + 64)."""
    freq = np.ones(256, np.uint16)
    freq[0] = 4096 - 255
    cdf = np.concatenate(([0], np.cumsum(freq.astype(np.int64))[:-1])).astype(np.uint16)
    sym = np.full((1024, 32), 5, np.uint8)
    with pytest.raises(RuntimeError, match="capacity"):
        oracle.encode_tiled_ilp2(sym, freq, cdf, 1024, 32)


def test_tile_height_must_be_multiple_of_16(oracle):
    sym = np.zeros((64, 32), np.uint8)
    f, c = _table(oracle, sym)
    with pytest.raises(RuntimeError):
        oracle.encode_tiled_ilp2(sym, f, c, 24, 32)


# ---- one stream per column and tile (the reference's first tiled format) ------------------------------------
@pytest.mark.parametrize("K,N,th,tw", [(80, 24, 32, 8), (700, 70, 256, 32), (1024, 64, 1024, 32), (50, 5, 64, 16)])
def test_one_stream_layout_round_trips_and_agrees_with_the_second_implementation(oracle, K, N, th, tw):
    """src/cuda/rans_kernels.cuh:316-391 + src/cuda/rans_ops.cu:522-566 + comp_inference/rans_triton.py:399-464:
    decode(encode(x)) == x; every stream ends on 2^16 with exactly its own bytes consumed; the numpy decoder
    written in the shape of the Triton kernel decodes the same bytes; the plain-integer encoder produces the same
    stream, state and zero-prefixed body column for every stream; offsets are the scan of depth * tw."""
    sym = zipf_bytes(K * N, 1.1, K + N).reshape(K, N)
    f, c = _table(oracle, sym)
    enc = oracle.encode_tiled_one(sym, f, c, th, tw)
    tiles_k, tiles_n = -(-K // th), -(-N // tw)
    assert enc.num_streams == tiles_k * tiles_n * tw and enc.states.size == enc.num_streams
    out, end, left = oracle.decode_tiled_one(enc.stream, enc.states, enc.tables, enc.slot_map, enc.tile_offsets,
                                             enc.tile_max_lens, K, N, th, tw, want_end=True)
    assert np.array_equal(out, sym)
    got = pyref.decode_tiled(enc.stream, enc.states, enc.tables, enc.slot_map, enc.tile_offsets, enc.tile_max_lens,
                             K, N, th, tw, halves=1)
    assert np.array_equal(got, sym)
    lane_col = (np.arange(enc.num_streams) // tw % tiles_n) * tw + np.arange(enc.num_streams) % tw
    live = lane_col < N
    assert (end[live] == L).all()
    pad_rows = np.repeat(enc.tile_max_lens, tw).astype(np.int64) - enc.sizes
    assert np.array_equal(left.astype(np.int64)[live], pad_rows[live] - 1)     # exactly its own bytes
    assert (enc.sizes[~live] == 0).all() and (enc.states[~live] == L).all()
    assert np.array_equal(enc.tile_offsets.astype(np.int64),
                          np.concatenate(([0], np.cumsum(enc.tile_max_lens.astype(np.int64) * tw)[:-1])))
    assert enc.stream.size == int((enc.tile_max_lens.astype(np.int64) * tw).sum())
    for sid in range(0, enc.num_streams, 3):
        t, q = divmod(sid, tw)
        tk, tn = divmod(t, tiles_n)
        col = tn * tw + q
        if col >= N:
            continue
        rows = [r for r in range(tk * th, tk * th + th) if r < K]
        x, emitted = pyref.encode_stream(sym[rows, col], f, c)
        assert enc.states[sid] == x and enc.sizes[sid] == len(emitted)
        depth = int(enc.tile_max_lens[t])
        body = enc.stream[enc.tile_offsets[t]:][: depth * tw].reshape(-1, tw)
        pad = depth - len(emitted)
        assert body[pad:, q].tolist() == emitted and not body[:pad, q].any()


def test_one_stream_layout_is_the_two_stream_layout_of_twice_the_columns(oracle):
    """A plane whose top and bottom half tiles are laid side by side: the one-stream coding of the [th/2, 2N]
    arrangement has, stream for stream, the states and bytes of the two-stream coding of the [th, N] plane --
    the two formats differ in how streams are grouped into bodies, not in the coder."""
    th, tw, N = 64, 8, 16
    sym = zipf_bytes(th * N, 1.2, 3).reshape(th, N)
    f, c = _table(oracle, sym)
    two = oracle.encode_tiled_ilp2(sym, f, c, th, tw)
    side = np.concatenate([np.concatenate([sym[: th // 2, tn * tw:(tn + 1) * tw], sym[th // 2:, tn * tw:(tn + 1) * tw]], 1)
                           for tn in range(N // tw)], 1)      # per column tile: [top | bottom]
    one = oracle.encode_tiled_one(np.ascontiguousarray(side), f, c, th // 2, 2 * tw)
    assert np.array_equal(one.states, two.states) and np.array_equal(one.sizes, two.sizes)
    assert np.array_equal(one.stream, two.stream) and np.array_equal(one.tile_max_lens, two.tile_max_lens)
