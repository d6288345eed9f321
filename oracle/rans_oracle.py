"""ctypes front end of the CPU oracle (``librans_oracle.so``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` as the checker.  The shipped package never imports it.

All arrays are numpy; every function mirrors one C entry point of ``rans_oracle.c`` (which
cites the reference lines it restates).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "librans_oracle.so")
_lib = None

_ERRORS = {1: "bad argument", 2: "stream outgrew the reference's per-stream capacity",
           3: "out of memory", 4: "corrupt input"}


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (a few seconds)."""
    src = os.path.join(_HERE, "rans_oracle.c")
    stale = (not os.path.exists(_LIB_PATH)) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src)
    if force or stale:
        subprocess.check_call(["make", "-C", _HERE, "-B", "librans_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.ro_interleaved_len.restype = C.c_uint64
        _lib.ro_flat_num_streams.restype = C.c_uint32
        _lib.ro_free.restype = None
    return _lib


def _p(a: np.ndarray | None):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"oracle {what}: {_ERRORS.get(rc, rc)}")


def _u8(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.uint8)


def _u16(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.uint16)


def _u32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.uint32)


# ------------------------------------------------------------------------------ planes
def split_bf16(w_bits: np.ndarray):
    w = _u16(w_bits)
    e = np.empty(w.shape, np.uint8)
    m = np.empty(w.shape, np.uint8)
    lib().ro_split_bf16(_p(w), C.c_uint64(w.size), _p(e), _p(m))
    return e, m


def merge_bf16(exp_plane: np.ndarray, man_plane: np.ndarray) -> np.ndarray:
    e, m = _u8(exp_plane), _u8(man_plane)
    assert e.shape == m.shape
    w = np.empty(e.shape, np.uint16)
    lib().ro_merge_bf16(_p(e), _p(m), C.c_uint64(e.size), _p(w))
    return w


def get_lut(data: np.ndarray):
    d = _u8(data).reshape(-1)
    f = np.empty(256, np.uint16)
    c = np.empty(256, np.uint16)
    _check(lib().ro_get_lut(_p(d), C.c_uint64(d.size), _p(f), _p(c)), "get_lut")
    return f, c


def build_tables(freq: np.ndarray, cdf: np.ndarray):
    t = np.zeros(256, np.uint32)
    s = np.zeros(4096, np.uint8)
    lib().ro_build_tables(_p(_u16(freq)), _p(_u16(cdf)), _p(t), _p(s))
    return t, s


# ------------------------------------------------------------------------------ results
@dataclass
class TiledResult:
    stream: np.ndarray
    states: np.ndarray
    sizes: np.ndarray
    tables: np.ndarray
    slot_map: np.ndarray
    tile_offsets: np.ndarray
    tile_max_lens: np.ndarray
    num_streams: int
    num_tiles_k: int
    num_tiles_n: int
    tile_height: int
    tile_width: int


@dataclass
class DenseResult:
    stream: np.ndarray
    states: np.ndarray
    sizes: np.ndarray
    tables: np.ndarray
    slot_map: np.ndarray
    stream_offsets: np.ndarray
    num_streams: int
    num_tiles_k: int
    num_tiles_n: int
    tile_height: int
    tile_width: int


@dataclass
class FlatResult:
    stream: np.ndarray
    states: np.ndarray
    sizes: np.ndarray
    tables: np.ndarray
    slot_map: np.ndarray
    checkpoints: np.ndarray
    num_streams: int


def _take_stream(ptr: C.c_void_p, n: int) -> np.ndarray:
    out = np.empty(n, np.uint8)
    if n:
        C.memmove(out.ctypes.data, ptr, n)
    lib().ro_free(ptr)
    return out


# ------------------------------------------------------------------------------ coders
def encode_tiled_ilp2(sym: np.ndarray, freq, cdf, th: int = 1024, tw: int = 32) -> TiledResult:
    sym = _u8(sym)
    K, N = sym.shape
    tk, tn = -(-K // th), -(-N // tw)
    T, S = tk * tn, tk * tn * 2 * tw
    states = np.empty(S, np.uint32)
    sizes = np.empty(S, np.uint32)
    offs = np.empty(T, np.uint32)
    lens = np.empty(T, np.uint32)
    sp = C.c_void_p()
    sl = C.c_uint64()
    _check(lib().ro_encode_tiled_ilp2(_p(sym), K, N, _p(_u16(freq)), _p(_u16(cdf)), th, tw,
                                      _p(states), _p(sizes), _p(offs), _p(lens),
                                      C.byref(sp), C.byref(sl)), "encode_tiled_ilp2")
    tables, slot_map = build_tables(freq, cdf)
    return TiledResult(_take_stream(sp, sl.value), states, sizes, tables, slot_map, offs, lens,
                       S, tk, tn, th, tw)


def decode_tiled_ilp2(stream, states, tables, slot_map, tile_offsets, tile_max_lens, K, N,
                      th=1024, tw=32, want_end=False):
    stream = _u8(stream)
    out = np.zeros((K, N), np.uint8)
    S = -(-K // th) * -(-N // tw) * 2 * tw
    states = _u32(states)
    assert states.size == S
    end = np.empty(S, np.uint32) if want_end else None
    left = np.empty(S, np.int32) if want_end else None
    _check(lib().ro_decode_tiled_ilp2(_p(stream), C.c_uint64(stream.size), _p(states),
                                      _p(_u32(tables)), _p(_u8(slot_map)), _p(_u32(tile_offsets)),
                                      _p(_u32(tile_max_lens)), K, N, th, tw, _p(out), _p(end),
                                      _p(left)), "decode_tiled_ilp2")
    return (out, end, left) if want_end else out


def encode_tiled_one(sym: np.ndarray, freq, cdf, th: int = 1024, tw: int = 32) -> TiledResult:
    """One stream per column and tile, packed into tile bodies of tw-byte rows (src/cuda/rans_kernels.cuh:316-391,
    src/cuda/rans_ops.cu:412-600)."""
    sym = _u8(sym)
    K, N = sym.shape
    tk, tn = -(-K // th), -(-N // tw)
    T, S = tk * tn, tk * tn * tw
    states = np.empty(S, np.uint32)
    sizes = np.empty(S, np.uint32)
    offs = np.empty(T, np.uint32)
    lens = np.empty(T, np.uint32)
    sp = C.c_void_p()
    sl = C.c_uint64()
    _check(lib().ro_encode_tiled_one(_p(sym), K, N, _p(_u16(freq)), _p(_u16(cdf)), th, tw,
                                     _p(states), _p(sizes), _p(offs), _p(lens),
                                     C.byref(sp), C.byref(sl)), "encode_tiled_one")
    tables, slot_map = build_tables(freq, cdf)
    return TiledResult(_take_stream(sp, sl.value), states, sizes, tables, slot_map, offs, lens,
                       S, tk, tn, th, tw)


def decode_tiled_one(stream, states, tables, slot_map, tile_offsets, tile_max_lens, K, N,
                     th=1024, tw=32, want_end=False):
    """comp_inference/rans_triton.py:399-464."""
    stream = _u8(stream)
    out = np.zeros((K, N), np.uint8)
    S = -(-K // th) * -(-N // tw) * tw
    states = _u32(states)
    assert states.size == S
    end = np.empty(S, np.uint32) if want_end else None
    left = np.empty(S, np.int32) if want_end else None
    _check(lib().ro_decode_tiled_one(_p(stream), C.c_uint64(stream.size), _p(states),
                                     _p(_u32(tables)), _p(_u8(slot_map)), _p(_u32(tile_offsets)),
                                     _p(_u32(tile_max_lens)), K, N, th, tw, _p(out), _p(end),
                                     _p(left)), "decode_tiled_one")
    return (out, end, left) if want_end else out


def encode_tiled_dense(sym: np.ndarray, freq, cdf, th: int = 1024, tw: int = 32) -> DenseResult:
    sym = _u8(sym)
    K, N = sym.shape
    tk, tn = -(-K // th), -(-N // tw)
    S = tk * tn * tw
    states = np.empty(S, np.uint32)
    sizes = np.empty(S, np.uint32)
    offs = np.empty(S, np.uint32)
    sp = C.c_void_p()
    sl = C.c_uint64()
    _check(lib().ro_encode_tiled_dense(_p(sym), K, N, _p(_u16(freq)), _p(_u16(cdf)), th, tw,
                                       _p(states), _p(sizes), _p(offs), C.byref(sp),
                                       C.byref(sl)), "encode_tiled_dense")
    tables, slot_map = build_tables(freq, cdf)
    return DenseResult(_take_stream(sp, sl.value), states, sizes, tables, slot_map, offs, S, tk, tn,
                       th, tw)


def decode_tiled_dense(stream, states, tables, slot_map, stream_offsets, stream_sizes, K, N,
                       th=1024, tw=32, want_end=False):
    stream = _u8(stream)
    out = np.zeros((K, N), np.uint8)
    S = -(-K // th) * -(-N // tw) * tw
    end = np.empty(S, np.uint32) if want_end else None
    left = np.empty(S, np.int32) if want_end else None
    _check(lib().ro_decode_tiled_dense(_p(stream), C.c_uint64(stream.size), _p(_u32(states)),
                                       _p(_u32(tables)), _p(_u8(slot_map)),
                                       _p(_u32(stream_offsets)), _p(_u32(stream_sizes)), K, N, th,
                                       tw, _p(out), _p(end), _p(left)), "decode_tiled_dense")
    return (out, end, left) if want_end else out


def flat_num_streams(K: int, N: int, min_block: int) -> int:
    return int(lib().ro_flat_num_streams(K, N, min_block))


def encode_flat(sym: np.ndarray, freq, cdf, min_block: int = 512) -> FlatResult:
    sym = _u8(sym)
    if sym.ndim == 1:
        sym = sym.reshape(-1, 1)
    K, N = sym.shape
    S = flat_num_streams(K, N, min_block)
    states = np.empty(S, np.uint32)
    sizes = np.empty(S, np.uint32)
    ck = np.empty(S * 128, np.uint64)
    sp = C.c_void_p()
    sl = C.c_uint64()
    _check(lib().ro_encode_flat(_p(sym), K, N, _p(_u16(freq)), _p(_u16(cdf)), min_block,
                                _p(states), _p(sizes), _p(ck), C.byref(sp), C.byref(sl)),
           "encode_flat")
    tables, slot_map = build_tables(freq, cdf)
    return FlatResult(_take_stream(sp, sl.value), states, sizes, tables, slot_map, ck, S)


def decode_flat_segmented(stream, states, sizes, tables, slot_map, K, N):
    stream = _u8(stream)
    states = _u32(states)
    out = np.zeros((K, N), np.uint8)
    _check(lib().ro_decode_flat_segmented(_p(stream), C.c_uint64(stream.size), _p(states),
                                          _p(_u32(sizes)), states.size, _p(_u32(tables)),
                                          _p(_u8(slot_map)), K, N, _p(out)), "decode_flat_segmented")
    return out


def decode_flat_strided(stream, states, sizes, tables, slot_map, out_len):
    stream = _u8(stream)
    states = _u32(states)
    out = np.zeros(out_len, np.uint8)
    _check(lib().ro_decode_flat_strided(_p(stream), C.c_uint64(stream.size), _p(states),
                                        _p(_u32(sizes)), states.size, _p(_u32(tables)),
                                        _p(_u8(slot_map)), C.c_uint64(out_len), _p(out)),
           "decode_flat_strided")
    return out


# ------------------------------------------------------------------------------ mantissa plane
def interleave_plane(plane: np.ndarray, th: int = 1024, tw: int = 32) -> np.ndarray:
    plane = _u8(plane)
    K, N = plane.shape
    out = np.empty(int(lib().ro_interleaved_len(K, N, th, tw)), np.uint8)
    lib().ro_interleave_plane(_p(plane), K, N, th, tw, _p(out))
    return out


def uninterleave_plane(tiled: np.ndarray, K: int, N: int, th: int = 1024, tw: int = 32):
    tiled = _u8(tiled).reshape(-1)
    out = np.empty((K, N), np.uint8)
    lib().ro_uninterleave_plane(_p(tiled), C.c_uint64(tiled.size), K, N, th, tw, _p(out))
    return out


# ------------------------------------------------------------------------------ GEMM / gather
def linear_reference_numerics(x_bits, w_bits, bias_bits=None, th=1024, split_k=8) -> np.ndarray:
    x, w = _u16(x_bits), _u16(w_bits)
    M, K = x.shape
    K2, N = w.shape
    assert K == K2
    out = np.empty((M, N), np.uint16)
    b = _u16(bias_bits) if bias_bits is not None else None
    lib().ro_linear_reference_numerics(_p(x), _p(w), _p(b), M, K, N, th, split_k, _p(out))
    return out


def linear_f32(x_bits, w_bits) -> np.ndarray:
    x, w = _u16(x_bits), _u16(w_bits)
    M, K = x.shape
    _, N = w.shape
    out = np.empty((M, N), np.float32)
    lib().ro_linear_f32(_p(x), _p(w), M, K, N, _p(out))
    return out


def embedding_gather(ids, enc: TiledResult, man_tiled, K, N) -> np.ndarray:
    ids = np.ascontiguousarray(ids, dtype=np.int64).reshape(-1)
    out = np.zeros((ids.size, N), np.uint16)
    _check(lib().ro_embedding_gather(_p(ids), ids.size, _p(enc.stream), _p(enc.states),
                                     _p(enc.tables), _p(enc.slot_map), _p(enc.tile_offsets),
                                     _p(enc.tile_max_lens), _p(_u8(man_tiled)), K, N,
                                     enc.tile_height, enc.tile_width, _p(out)), "embedding_gather")
    return out


# ------------------------------------------------------------------------------ convenience
def compress_bf16(w_bits: np.ndarray, th: int = 1024, tw: int = 32):
    """bf16 bit patterns [K,N] -> (TiledResult for the exponent plane, tiled sign|mantissa)."""
    e, m = split_bf16(w_bits)
    f, c = get_lut(e)
    return encode_tiled_ilp2(e, f, c, th, tw), interleave_plane(m, th, tw)


def decompress_bf16(enc: TiledResult, man_tiled, K, N) -> np.ndarray:
    e = decode_tiled_ilp2(enc.stream, enc.states, enc.tables, enc.slot_map, enc.tile_offsets,
                          enc.tile_max_lens, K, N, enc.tile_height, enc.tile_width)
    m = uninterleave_plane(man_tiled, K, N, enc.tile_height, enc.tile_width)
    return merge_bf16(e, m)
