"""Loader of libcomp_inference_hip.so and the small amount of glue every op needs.

There is no CPU or eager fallback: if the shared library is missing, or the current device
is not a gfx950, the ops raise.
"""
from __future__ import annotations

import ctypes as C
import os

import torch

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libcomp_inference_hip.so")
_lib = None
_device_ok: set[int] = set()


class Tiling(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in (
        "K", "N", "tile_height", "tile_width", "num_tiles_k", "num_tiles_n", "num_tiles",
        "streams_per_tile", "num_streams", "capacity")]


class TiledWeight(C.Structure):
    """ci_tiled_weight: a compressed weight with the length of every array (include/comp_inference_hip.h)."""
    _fields_ = [("K", C.c_uint32), ("N", C.c_uint32), ("tile_height", C.c_uint32), ("tile_width", C.c_uint32),
                ("d_stream", C.c_void_p), ("stream_len", C.c_uint64),
                ("d_states", C.c_void_p), ("n_states", C.c_uint64),
                ("d_tables", C.c_void_p), ("d_slot_map", C.c_void_p),
                ("d_tile_offsets", C.c_void_p), ("d_tile_max_lens", C.c_void_p), ("n_tiles", C.c_uint64),
                ("d_man_tiled", C.c_void_p), ("man_len", C.c_uint64),
                ("d_checkpoints", C.c_void_p), ("checkpoint_bytes", C.c_uint64), ("segments", C.c_uint32),
                ("d_slot_table", C.c_void_p), ("slot_table_bytes", C.c_uint64), ("max_window_rows", C.c_uint32)]


SLOT_TABLE_BYTES = 32768


def tiled_weight(K, N, tile_k, tile_n, stream, states, tables, slot_map, tile_offsets, tile_max_lens, man,
                 checkpoints=None, segments=1, slot_table=None, max_window_rows=0) -> TiledWeight:
    """Descriptor over device tensors (which the caller keeps alive for as long as it is used)."""
    w = TiledWeight()
    w.K, w.N, w.tile_height, w.tile_width = int(K), int(N), int(tile_k), int(tile_n)
    w.d_stream, w.stream_len = stream.data_ptr() if stream.numel() else None, stream.numel()
    w.d_states, w.n_states = states.data_ptr(), states.numel()
    w.d_tables, w.d_slot_map = tables.data_ptr(), slot_map.data_ptr()
    w.d_tile_offsets, w.d_tile_max_lens = tile_offsets.data_ptr(), tile_max_lens.data_ptr()
    w.n_tiles = min(tile_offsets.numel(), tile_max_lens.numel())
    w.d_man_tiled, w.man_len = (man.data_ptr(), man.numel()) if man is not None else (None, 0)
    if checkpoints is not None and segments > 1:
        w.d_checkpoints, w.checkpoint_bytes, w.segments = checkpoints.data_ptr(), checkpoints.numel() * 8, int(segments)
    else:
        w.d_checkpoints, w.checkpoint_bytes, w.segments = None, 0, 1
    if slot_table is not None:
        w.d_slot_table, w.slot_table_bytes = slot_table.data_ptr(), slot_table.numel() * slot_table.element_size()
    else:
        w.d_slot_table, w.slot_table_bytes = None, 0
    w.max_window_rows = int(max_window_rows)
    return w


def lib() -> C.CDLL:
    """The shared library; raises RuntimeError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m comp_inference_amd.build` "
                "(hipcc, gfx950). The HIP extension is the only implementation of these ops.")
        _lib = C.CDLL(LIB_PATH)
        _lib.ci_last_error.restype = C.c_char_p
        _lib.ci_encode_scratch_bytes.restype = C.c_size_t
        _lib.ci_fused_linear_workspace_bytes.restype = C.c_size_t
        _lib.ci_fused_embedding_workspace_bytes.restype = C.c_size_t
        _lib.ci_fused_linear_transposed_workspace_bytes.restype = C.c_size_t
        _lib.ci_fused_linear_workspace_bytes_segmented.restype = C.c_size_t
        _lib.ci_checkpoint_bytes.restype = C.c_size_t
        _lib.ci_fused_embedding_workspace_bytes_segmented.restype = C.c_size_t
        _lib.ci_suggest_segments.restype = C.c_uint32
    return _lib


def check(rc: int) -> None:
    """0 -> return; anything else -> RuntimeError carrying the library's message (the reference
    surfaces the same conditions as RuntimeError through pybind11)."""
    if rc != 0:
        raise RuntimeError(lib().ci_last_error().decode() or f"comp_inference_hip error {rc}")


def require_device(t: torch.Tensor) -> None:
    """Ops run on gfx950 tensors only."""
    if not t.is_cuda:
        raise RuntimeError("tensor must be on the GPU")  # src/python_bindings.cpp:68-69
    idx = t.device.index if t.device.index is not None else torch.cuda.current_device()
    if idx not in _device_ok:
        with torch.cuda.device(idx):
            check(lib().ci_check_device())
        _device_ok.add(idx)


def ptr(t: torch.Tensor | None) -> C.c_void_p:
    return C.c_void_p(t.data_ptr()) if t is not None and t.numel() else C.c_void_p(0)


def stream_handle(device: torch.device) -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def as_u32(t: torch.Tensor, device) -> torch.Tensor:
    """uint32/int32 metadata tensors are accepted interchangeably (the reference's callers pass
    both, comp_inference/comp_inference.py:636-642 vs comp_inference/rans_saving.py:396-404)."""
    if t.dtype not in (torch.uint32, torch.int32):
        t = t.to(torch.int64).to(torch.uint32) if t.dtype != torch.uint32 else t
    return t.to(device).contiguous()


def as_u8(t: torch.Tensor, device) -> torch.Tensor:
    if t.dtype != torch.uint8:
        t = t.to(torch.uint8)
    return t.to(device).contiguous()


def check_tiled_operands(rows: int, cols: int, tile_k: int, tile_n: int, initial_states, tables, slot_map, meta0, meta1,
                         dense: bool, one: bool = False) -> None:
    """The kernels index these arrays by tile and stream without a bound of their own: a short one would be
    read past its end.  Same condition and exception as the reference's decoder
    (comp_inference/rans_triton.py:141-144, :482-487), applied to every operand and every op.
    `dense`: one stream per column with per-stream offsets and sizes; `one`: one stream per column in
    tile bodies (per-tile offsets and depths); neither: two streams per column in tile bodies."""
    tiles = (-(-rows // tile_k)) * (-(-cols // tile_n))
    streams = tiles * tile_n * (1 if dense or one else 2)
    if initial_states.numel() != streams:
        raise ValueError(f"Initial states size mismatch. Expected {streams}")
    per_meta = streams if dense else tiles
    if meta0.numel() != per_meta or meta1.numel() != per_meta:
        what = "stream offsets / sizes" if dense else "tile offsets / max lens"
        raise ValueError(f"{what} size mismatch. Expected {per_meta}")
    if tables.numel() != 256 or slot_map.numel() != 4096:
        raise ValueError("tables must hold 256 entries and slot_map 4096")

