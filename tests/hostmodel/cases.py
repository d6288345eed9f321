"""One call of each operator of the library on the host model, compared with the oracle: the building blocks of the
test_hostmodel_* files.  Every function raises on a difference, on an error of the entry point, and on anything the
model reports (an address outside an array, a register used before its load was waited for, ...)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from oracle import rans_oracle as ro
from tests.hostmodel.model import Model, bf16_bits_to_f32, f32_to_bf16_bits


# ---- weights whose exponent planes leave the well-trodden paths -----------------------------------------------------
def weight_kind(rng: np.random.Generator, K: int, N: int, kind: str) -> np.ndarray:
    """bf16 bit patterns [K, N].  normal: N(0, 0.02); constant: one exponent throughout (streams almost without
    bytes); sparse: 90 % zeros; wide: exponents spread over thirty binades (deep tile bodies, rare symbols: two-byte
    renormalisations); mixed: columns of very different compressibility inside one tile (windows far apart)."""
    if kind == "normal":
        w = rng.standard_normal((K, N), dtype=np.float32) * 0.02
    elif kind == "constant":
        w = (1.0 + rng.random((K, N), dtype=np.float32) * 0.99).astype(np.float32) * np.where(rng.random((K, N)) < 0.5, -1, 1)
    elif kind == "sparse":
        w = rng.standard_normal((K, N), dtype=np.float32) * 0.02 * (rng.random((K, N)) < 0.1)
    elif kind == "wide":
        w = rng.standard_normal((K, N), dtype=np.float32) * np.exp2(rng.integers(-20, 10, (K, N))).astype(np.float32)
    elif kind == "mixed":
        w = rng.standard_normal((K, N), dtype=np.float32) * 0.02
        wide = rng.standard_normal((K, N), dtype=np.float32) * np.exp2(rng.integers(-20, 10, (K, N))).astype(np.float32)
        w = np.where((np.arange(N) % 5 == 0)[None, :], wide, w)
    else:
        raise ValueError(kind)
    return f32_to_bf16_bits(w.astype(np.float32))


KINDS = ("normal", "constant", "sparse", "wide", "mixed")


def compress(bits: np.ndarray, th: int, tw: int = 32):
    return ro.compress_bf16(bits, th, tw)


def _ws(m: Model, nbytes: int):
    return m.empty(max(int(nbytes), 16), np.uint8), C.c_size_t(int(nbytes))


# ---- stand-alone decode ---------------------------------------------------------------------------------------------
def decode(m: Model, bits, th, segments=1, merge=False, expect_kernel=None):
    K, N = bits.shape
    enc, man = compress(bits, th)
    w, keep = m.weight(enc, man, K, N, segments=segments)
    m.clear()
    if merge:
        out = m.empty((K, N), np.uint16)
        m.call("ci_decode_tiled", C.byref(w), None, out.p, None)
        assert np.array_equal(out.get(), bits), "decoded bf16 differs"
    else:
        out = m.empty((K, N), np.uint8)
        m.call("ci_decode_tiled", C.byref(w), out.p, None, None)
        assert np.array_equal(out.get(), ro.split_bf16(bits)[0]), "decoded exponent plane differs"
    if expect_kernel:
        assert any(expect_kernel in k for k in m.launches()), (expect_kernel, m.launches())
    return m.launches()


# ---- fused linear ---------------------------------------------------------------------------------------------------
def linear(m: Model, bits, xb, th, segments=1, slot_table=False, window_rows=False, wide=False, bias=None,
           noalloc=False, expect_kernel=None, x_pad=0, check_twin=True, partials_only=False):
    """out = x W through ci_fused_linear_tiled (or its no-allocation variant): within 1e-2 of the fp32 product on the
    oracle-decoded weight, and bit for bit the same contraction on the plain weight.  partials_only: the workspace has
    room for the partial sums the plan needs and not for the fragment copy of x (a caller that sized it so): the
    kernels then read the rows of x where they lie."""
    K, N = bits.shape
    M = xb.shape[0]
    enc, man = compress(bits, th)
    assert np.array_equal(ro.decompress_bf16(enc, man, K, N), bits)
    w, keep = m.weight(enc, man, K, N, segments=segments, slot_table=slot_table, window_rows=window_rows)
    xs = K + x_pad  # row stride of x
    xfull = np.zeros((M, xs), np.uint16)
    xfull[:, :K] = xb
    x, out = m.dev(xfull), m.empty((M, N), np.uint16)
    b = m.dev(bias) if bias is not None else None
    nb = m.lib.ci_fused_linear_workspace_bytes_segmented(M, K, N, th, 32, 0, segments)
    if partials_only:
        # what the query adds for the fragment copy: whole passes of 4 or 8 groups of 32 rows above 64 rows, else pairs
        # of groups above 32 rows, else one group (from 17 rows on, K a multiple of 8)
        groups = -(-M // 32)
        groups = -(-groups // (4 if M <= 128 else 8)) * (4 if M <= 128 else 8) if M > 64 else (2 * -(-M // 64) if M > 32 else 1)
        frag = groups * 32 * K * 2 if (M >= 17 and K % 8 == 0) else 0
        assert nb >= frag
        nb -= frag
    ws, ws_n = _ws(m, nb)
    m.lib.ci_fused_linear_wide_rows(1 if wide else 0)
    m.clear()
    try:
        if noalloc:
            m.call("ci_fused_linear_tiled_noalloc", C.byref(w), x.p, M, xs, b.p if b else None, out.p, N, None)
        else:
            m.call("ci_fused_linear_tiled", C.byref(w), x.p, M, xs, b.p if b else None, out.p, N, ws.p, ws_n, None)
        launches = m.launches()
        if check_twin:
            out2, wd = m.empty((M, N), np.uint16), m.dev(bits)
            m.call("ci_plain_linear_same_order", x.p, M, K, N, xs, wd.p, th, 32, segments, b.p if b else None, out2.p, N,
                   ws.p, ws_n, None)
            assert np.array_equal(out.get(), out2.get()), "fused linear differs from the same contraction on the plain weight"
    finally:
        m.lib.ci_fused_linear_wide_rows(0)
    want = ro.linear_f32(xb, bits)
    if bias is not None:
        want = want + bf16_bits_to_f32(bias)[None, :]
    got = bf16_bits_to_f32(out.get())
    finite = np.isfinite(want)
    tol = 1e-2 * max(1.0, float(np.abs(want[finite]).max()))  # (weights of the wide kinds give sums far above 1)
    assert np.allclose(got[finite], want[finite], atol=tol, rtol=1e-2), f"fused linear: max error {np.abs(got - want)[finite].max()}"
    if expect_kernel:
        assert any(expect_kernel in k for k in launches), (expect_kernel, launches)
    return launches


# ---- fused gather ---------------------------------------------------------------------------------------------------
def gather(m: Model, bits, ids, th, segments=1, slot_table=False, expect_kernel=None):
    K, N = bits.shape
    enc, man = compress(bits, th)
    w, keep = m.weight(enc, man, K, N, segments=segments, slot_table=slot_table)
    ids = np.ascontiguousarray(ids, np.int64)
    d_ids, out = m.dev(ids), m.empty((ids.size, N), np.uint16)
    nb = m.lib.ci_fused_embedding_workspace_bytes_segmented(ids.size, K, th, segments)
    ws, ws_n = _ws(m, nb)
    m.clear()
    m.call("ci_fused_embedding_tiled", C.byref(w), d_ids.p, ids.size, out.p, N, ws.p, ws_n, None)
    want = np.zeros((ids.size, N), np.uint16)
    ok = (ids >= 0) & (ids < K)
    want[ok] = bits[ids[ok]]
    assert np.array_equal(out.get(), want), "gathered rows differ from table[ids]"
    if expect_kernel:
        assert any(expect_kernel in k for k in m.launches()), (expect_kernel, m.launches())
    return m.launches()


def zipf_ids(rng, K, n, s=1.1):
    p = 1.0 / np.arange(1, K + 1) ** s
    p /= p.sum()
    return rng.choice(K, n, p=p).astype(np.int64)


# ---- LM head (weight stored [V, H]) -----------------------------------------------------------------------------------
def lm_head(m: Model, bits, xb, th, segments=1, slot_table=False, window_rows=False, matrix_sums=False, bias=None,
            expect_kernel=None, check_twin=True):
    V, H = bits.shape
    M = xb.shape[0]
    enc, man = compress(bits, th)
    w, keep = m.weight(enc, man, V, H, segments=segments, slot_table=slot_table, window_rows=window_rows)
    x, out = m.dev(xb), m.empty((M, V), np.uint16)
    b = m.dev(bias) if bias is not None else None
    nb = m.lib.ci_fused_linear_transposed_workspace_bytes(M, H, V, 32)
    ws, ws_n = _ws(m, nb)
    m.lib.ci_fused_linear_transposed_matrix_sums(1 if matrix_sums else 0)
    m.clear()
    try:
        m.call("ci_fused_linear_transposed_tiled", C.byref(w), x.p, M, H, b.p if b else None, out.p, V, ws.p, ws_n, None)
    finally:
        m.lib.ci_fused_linear_transposed_matrix_sums(0)
    launches = m.launches()
    if check_twin:
        out2, wd = m.empty((M, V), np.uint16), m.dev(bits)
        m.call("ci_plain_linear_transposed_same_order", x.p, M, H, V, H, wd.p, th, 32, b.p if b else None, out2.p, V, ws.p,
               ws_n, None)
        assert np.array_equal(out.get(), out2.get()), "LM head differs from the same contraction on the plain weight"
    want = ro.linear_f32(xb, np.ascontiguousarray(bits.T))
    if bias is not None:
        want = want + bf16_bits_to_f32(bias)[None, :]
    got = bf16_bits_to_f32(out.get())
    finite = np.isfinite(want)
    tol = 1e-2 * max(1.0, float(np.abs(want[finite]).max()))
    assert np.allclose(got[finite], want[finite], atol=tol, rtol=1e-2), f"LM head: max error {np.abs(got - want)[finite].max()}"
    if expect_kernel:
        assert any(expect_kernel in k for k in launches), (expect_kernel, launches)
    return launches


# ---- encoders ---------------------------------------------------------------------------------------------------------
class Tiling(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("K", "N", "tile_height", "tile_width", "num_tiles_k", "num_tiles_n", "num_tiles",
                                          "streams_per_tile", "num_streams", "capacity")]


def encode(m: Model, exp_plane, th, tw, layout="ilp2"):
    """The library's encoder + packer of one layout on the model against the oracle's, every output array compared."""
    K, N = exp_plane.shape
    f, c = ro.get_lut(exp_plane)
    t = Tiling()
    m.call("ci_tiling_init", C.byref(t), K, N, th, tw, 1 if layout == "ilp2" else 0)
    nb = m.lib.ci_encode_scratch_bytes(t.num_streams, t.capacity)
    sym, scratch = m.dev(exp_plane), m.empty(nb, np.uint8)
    states, sizes = m.empty(t.num_streams, np.uint32), m.empty(t.num_streams, np.uint32)
    f16, c16 = np.ascontiguousarray(f, np.uint16), np.ascontiguousarray(c, np.uint16)
    fp, cp = f16.ctypes.data_as(C.c_void_p), c16.ctypes.data_as(C.c_void_p)
    n = C.c_uint64(0)
    m.clear()
    oracle_encoder = {"ilp2": ro.encode_tiled_ilp2, "one": ro.encode_tiled_one, "dense": ro.encode_tiled_dense}[layout]
    try:
        want = oracle_encoder(exp_plane, f, c, th, tw)
    except RuntimeError as e:
        if "outgrew" not in str(e):
            raise
        # a stream longer than the capacity the reference reserves: the library must refuse the input too
        meta = [m.empty(max(t.num_streams, t.num_tiles), np.uint32).p for _ in range(2 if layout != "dense" else 1)]
        rc = getattr(m.lib, f"ci_encode_tiled_{layout}")(sym.p, C.byref(t), fp, cp, scratch.p, C.c_size_t(nb), states.p, sizes.p,
                                                         *meta, C.byref(n), None)
        assert rc != 0 and m.violations() == [], "the oracle refuses this input (capacity), the library encoded it"
        raise
    if layout == "dense":
        offs = m.empty(t.num_streams, np.uint32)
        m.call("ci_encode_tiled_dense", sym.p, C.byref(t), fp, cp, scratch.p, C.c_size_t(nb), states.p, sizes.p, offs.p,
               C.byref(n), None)
        stream = m.empty(n.value, np.uint8)
        m.call("ci_pack_tiled_dense", scratch.p, C.byref(t), sizes.p, offs.p, stream.p, n, None)
        assert np.array_equal(offs.get(), want.stream_offsets)
    else:
        offs, lens = m.empty(t.num_tiles, np.uint32), m.empty(t.num_tiles, np.uint32)
        m.call(f"ci_encode_tiled_{layout}", sym.p, C.byref(t), fp, cp, scratch.p, C.c_size_t(nb), states.p, sizes.p, offs.p,
               lens.p, C.byref(n), None)
        stream = m.empty(n.value, np.uint8)
        m.call(f"ci_pack_tiled_{layout}", scratch.p, C.byref(t), sizes.p, offs.p, lens.p, stream.p, n, None)
        assert np.array_equal(offs.get(), want.tile_offsets) and np.array_equal(lens.get(), want.tile_max_lens)
    assert n.value == want.stream.size and np.array_equal(stream.get(), want.stream), "packed stream differs from the oracle's"
    assert np.array_equal(states.get(), want.states) and np.array_equal(sizes.get(), want.sizes)
    return want


# ---- the operators on the other layouts (one thread per stream) ---------------------------------------------------------
def other_layout_ops(m: Model, bits, xb, ids, th, tw, layout, damage=None):
    """decode, fused linear, gather and LM head of the one-stream-per-column layout ("one") or the dense layout
    ("dense") or another tile width of the default layout ("ilp2"), against the oracle.  `damage(enc)` may overwrite
    the encoder's arrays first (same lengths): the operators must then still return without anything the model
    reports, and their results are not looked at."""
    K, N = bits.shape
    e, man_plane = ro.split_bf16(bits)
    f, c = ro.get_lut(e)
    man = ro.interleave_plane(man_plane, th, tw)
    enc = {"one": ro.encode_tiled_one, "dense": ro.encode_tiled_dense, "ilp2": ro.encode_tiled_ilp2}[layout](e, f, c, th, tw)
    intact = damage is None
    if not intact:
        damage(enc)
    d = dict(stream=m.dev(enc.stream), states=m.dev(enc.states), tables=m.dev(enc.tables), slot_map=m.dev(enc.slot_map), man=m.dev(man))
    if layout == "dense":
        sizes = np.diff(np.append(enc.stream_offsets, enc.stream.size).astype(np.int64)).astype(np.uint32)
        meta = (m.dev(enc.stream_offsets), m.dev(sizes))
    else:
        meta = (m.dev(enc.tile_offsets), m.dev(enc.tile_max_lens))
    common = (d["stream"].p, C.c_uint64(enc.stream.size), d["states"].p, d["tables"].p, d["slot_map"].p, meta[0].p, meta[1].p)
    suffix = {"one": "one", "dense": "dense", "ilp2": "ilp2"}[layout]
    m.clear()
    # decode: exponent plane, then merged bf16
    out = m.empty((K, N), np.uint8)
    m.call(f"ci_decode_tiled_{suffix}", *common, K, N, th, tw, out.p, None, None, None)
    assert not intact or np.array_equal(out.get(), e), f"{layout}: decoded plane differs"
    outb = m.empty((K, N), np.uint16)
    m.call(f"ci_decode_tiled_{suffix}", *common, K, N, th, tw, None, d["man"].p, outb.p, None)
    assert not intact or np.array_equal(outb.get(), bits), f"{layout}: decoded bf16 differs"
    # fused linear
    M = xb.shape[0]
    x, y = m.dev(xb), m.empty((M, N), np.uint16)
    nb = m.lib.ci_fused_linear_workspace_bytes(M, K, N, th, tw, 0 if layout == "ilp2" else 1)
    ws, ws_n = _ws(m, nb)
    m.call(f"ci_fused_linear_{suffix}", x.p, M, K, N, K, *common, d["man"].p, th, tw, None, y.p, N, ws.p, ws_n, None)
    want = ro.linear_f32(xb, bits)
    assert not intact or np.allclose(bf16_bits_to_f32(y.get()), want, atol=1e-2, rtol=1e-2), f"{layout}: fused linear"
    # gather
    ids = np.ascontiguousarray(ids, np.int64)
    g = m.empty((ids.size, N), np.uint16)
    if layout == "ilp2":
        nbe = m.lib.ci_fused_embedding_workspace_bytes(ids.size, K, th)
        wse, wse_n = _ws(m, nbe)
        m.call("ci_fused_embedding_ilp2", m.dev(ids).p, ids.size, *common, d["man"].p, K, N, th, tw, g.p, N, wse.p, wse_n, None)
    else:
        m.call(f"ci_fused_embedding_{suffix}", m.dev(ids).p, ids.size, *common, d["man"].p, K, N, th, tw, g.p, N, None)
    wantg = np.zeros((ids.size, N), np.uint16)
    ok = (ids >= 0) & (ids < K)
    wantg[ok] = bits[ids[ok]]
    assert not intact or np.array_equal(g.get(), wantg), f"{layout}: gathered rows differ"
    # LM head: the same arrays read as a [V = K, H = N] table
    xh = xb[:, :N] if xb.shape[1] >= N else np.resize(xb, (M, N))
    xh = np.ascontiguousarray(xh)
    z = m.empty((M, K), np.uint16)
    nbt = m.lib.ci_fused_linear_transposed_workspace_bytes(M, N, K, tw)
    wst, wst_n = _ws(m, nbt)
    m.call(f"ci_fused_linear_transposed_{suffix}", m.dev(xh).p, M, N, K, N, *common, d["man"].p, th, tw, None, z.p, K, wst.p,
           wst_n, None)
    wantz = ro.linear_f32(xh, np.ascontiguousarray(bits.T))
    assert not intact or np.allclose(bf16_bits_to_f32(z.get()), wantz, atol=1e-2, rtol=1e-2), f"{layout}: LM head"
    return m.launches()
