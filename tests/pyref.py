"""A second, independent statement of the tiled two-streams-per-column format, written with numpy
vector operations over the lanes of a tile (the shape of the reference's Triton decoder,
comp_inference/rans_triton.py:34-119) and plain Python integers for the encoder of one stream
(src/cuda/rans_kernels.cuh:123-151).  Used only to cross-check the C oracle: an indexing or
ordering slip in one of the two would not be repeated in the other."""
import numpy as np

L = 1 << 16
M = 1 << 12


def encode_stream(symbols, freq, cdf):
    """Symbols in the order they are to be decoded; returns (final_state, bytes in emission order)."""
    x, out = L, []
    for s in reversed(list(symbols)):
        f, c = int(freq[s]), int(cdf[s])
        x_max = ((L >> 12) << 8) * f
        while x >= x_max:
            out.append(x & 0xFF)
            x >>= 8
        x = ((x // f) << 12) + (x % f) + c
    return x, out


def decode_tiled(stream, states, tables, slot_map, tile_offsets, tile_max_lens, K, N, th, tw, halves=2):
    """halves = 2: two streams per column and tile (rows [0, th/2) and [th/2, th)); halves = 1: one stream over
    the whole tile height (comp_inference/rans_triton.py:399-464)."""
    tiles_k, tiles_n = -(-K // th), -(-N // tw)
    half, spt = th // halves, halves * tw
    out = np.zeros((K, N), np.uint8)
    freq = (tables & 0xFFFF).astype(np.int64)
    cdf = (tables >> 16).astype(np.int64)
    lane = np.arange(spt)
    for t in range(tiles_k * tiles_n):
        tk, tn = divmod(t, tiles_n)
        x = states[t * spt:(t + 1) * spt].astype(np.int64)
        r = np.full(spt, int(tile_max_lens[t]) - 1, np.int64)
        base = int(tile_offsets[t])
        col = tn * tw + lane % tw
        for i in range(half):
            row = tk * th + i + (lane // tw) * half
            live = (col < N) & (row < K)
            slot = x & (M - 1)
            s = slot_map[slot].astype(np.int64)
            out[row[live], col[live]] = s[live]
            nx = freq[s] * (x >> 12) + slot - cdf[s]
            x = np.where(live, nx, x)
            for _ in range(2):
                need = live & (x < L) & (r >= 0)
                if len(stream):
                    b = stream[np.clip(base + r * spt + lane, 0, len(stream) - 1)].astype(np.int64)
                else:  # nothing was emitted (a constant plane): no lane can need a byte
                    b = np.zeros(spt, np.int64)
                x = np.where(need, (x << 8) | b, x)
                r = r - need
    return out
