#!/usr/bin/env python3
"""Writes tests/golden/small_formats.npz: one small bf16 weight in every stored layout.

The reference holds no golden vectors for this path (its tests check round trips only), so these
are made here: the default-layout stream comes from the pure-Python integer encoder of
tests/pyref.py and must equal the C oracle's byte for byte before anything is written, and so does the
one-stream-per-column stream; the dense and flat layouts come from the oracle and must round-trip.  The
file pins today's agreed bytes against later changes of the oracle, the host code and the HIP encoder
alike.

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))                   # tests/
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))  # repository root

import pyref  # noqa: E402
from oracle import rans_oracle as ro  # noqa: E402

K, N, TH, TW = 160, 72, 64, 32  # ragged in both directions: 3 x 3 tiles, the last ones partly empty


def python_encode_tiled(exp, freq, cdf, halves=2):
    """A tiled layout from first principles: per-stream Python encoder, bottom-aligned pack.  halves = 2: the
    default layout (two streams per column and tile); halves = 1: one stream per column over the tile's height."""
    tiles_k, tiles_n, half = -(-K // TH), -(-N // TW), TH // halves
    states, sizes, bodies, offsets, depths = [], [], [], [], []
    total = 0
    for tk in range(tiles_k):
        for tn in range(tiles_n):
            streams = []
            for q in range(halves * TW):
                col, r0 = tn * TW + q % TW, tk * TH + (q // TW) * half
                rows = [r for r in range(r0, r0 + half) if r < K] if col < N else []
                x, out = pyref.encode_stream([int(exp[r, col]) for r in rows], freq, cdf)
                streams.append(out)
                states.append(x)
                sizes.append(len(out))
            depth = max(len(s) for s in streams)
            body = np.zeros((depth, halves * TW), np.uint8)
            for q, s in enumerate(streams):
                if s:
                    body[depth - len(s):, q] = s
            offsets.append(total)
            depths.append(depth)
            total += body.size
            bodies.append(body.reshape(-1))
    return (np.concatenate(bodies), np.array(states, np.uint32), np.array(sizes, np.uint32),
            np.array(offsets, np.uint32), np.array(depths, np.uint32))


def main():
    rng = np.random.default_rng(20240607)
    w = (rng.standard_normal((K, N)).astype(np.float32) * 0.02)
    bits = (w.view(np.uint32) >> 16).astype(np.uint16)  # truncation is fine: any bf16 pattern will do
    exp, man = ro.split_bf16(bits)
    freq, cdf = ro.get_lut(exp)
    tables, slot_map = ro.build_tables(freq, cdf)

    t = ro.encode_tiled_ilp2(exp, freq, cdf, TH, TW)
    stream, states, sizes, offsets, depths = python_encode_tiled(exp, freq, cdf)
    assert np.array_equal(stream, t.stream) and np.array_equal(states, t.states)
    assert np.array_equal(sizes, t.sizes) and np.array_equal(offsets, t.tile_offsets)
    assert np.array_equal(depths, t.tile_max_lens)
    assert np.array_equal(pyref.decode_tiled(stream, states, tables, slot_map, offsets, depths, K, N, TH, TW), exp)

    o = ro.encode_tiled_one(exp, freq, cdf, TH, TW)
    one = python_encode_tiled(exp, freq, cdf, halves=1)
    for mine, theirs in zip(one, (o.stream, o.states, o.sizes, o.tile_offsets, o.tile_max_lens)):
        assert np.array_equal(mine, theirs)
    assert np.array_equal(pyref.decode_tiled(*one[:2], tables, slot_map, *one[3:], K, N, TH, TW, halves=1), exp)

    d = ro.encode_tiled_dense(exp, freq, cdf, TH, TW)
    d_sizes = np.diff(np.concatenate([d.stream_offsets, [d.stream.size]])).astype(np.uint32)
    assert np.array_equal(ro.decode_tiled_dense(d.stream, d.states, tables, slot_map, d.stream_offsets, d_sizes,
                                                K, N, TH, TW), exp)
    f = ro.encode_flat(exp, freq, cdf, 512)
    assert np.array_equal(ro.decode_flat_segmented(f.stream, f.states, f.sizes, tables, slot_map, K, N), exp)

    np.savez_compressed(
        os.path.join(HERE, "small_formats.npz"), shape=np.array([K, N, TH, TW], np.uint32), w_bits=bits, exp=exp,
        man=man, man_tiled=ro.interleave_plane(man, TH, TW), freq=freq, cdf=cdf, tables=tables, slot_map=slot_map,
        ilp2_stream=stream, ilp2_states=states, ilp2_sizes=sizes, ilp2_tile_offsets=offsets,
        ilp2_tile_max_lens=depths, one_stream=one[0], one_states=one[1], one_sizes=one[2], one_tile_offsets=one[3],
        one_tile_max_lens=one[4], dense_stream=d.stream, dense_states=d.states,
        dense_stream_offsets=d.stream_offsets, flat_stream=f.stream, flat_states=f.states, flat_sizes=f.sizes)
    print("wrote small_formats.npz:", stream.size, "bytes of default-layout stream,", one[0].size, "one stream per column,",
          d.stream.size, "dense,", f.stream.size, "flat")


if __name__ == "__main__":
    main()
