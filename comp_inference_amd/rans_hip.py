"""Stand-alone rANS decode ops on the GPU.

Same call signatures as the reference's Triton entry points
(comp_inference/rans_triton.py:122-168, :243-271); the kernels underneath are HIP
(csrc/decode.hip, csrc/legacy.hip).  All ops run on the current torch stream and do not wait.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from ._lib import check, lib, ptr


def _tiles(K: int, N: int, tile_k: int, tile_n: int):
    return (N + tile_n - 1) // tile_n, (K + tile_k - 1) // tile_k


def _checked_checkpoints(checkpoints, segments, K, N, tile_k, tile_n, dev):
    """-> (device tensor or None, segment count) for the segmented entry points."""
    segments = int(segments) if checkpoints is not None else 1
    if segments <= 1:
        return None, 1
    ck = checkpoints.to(dev).contiguous()
    if ck.dtype != torch.int64 or ck.numel() * 8 != lib().ci_checkpoint_bytes(K, N, int(tile_k), int(tile_n), segments):
        raise RuntimeError("checkpoints do not belong to this shape, tiling and segment count")
    return ck, segments


def rans_decomp_tiled(compressed_streams, initial_states, tables, slot_map, output_shape,
                      tile_offsets, tile_max_lens, tile_k=1024, tile_n=32, mantissas=None, out=None,
                      checkpoints=None, segments=1):
    """Decode the tiled two-streams-per-column format into the exponent plane u8[K,N]
    (comp_inference/rans_triton.py:122-168).  With `mantissas` (the tile-interleaved sign|mantissa
    plane) the bf16 weight [K,N] is returned instead, merged in the same kernel.  `out`: a contiguous
    GPU tensor of that shape and dtype to decode into (not in the reference's signature).
    `checkpoints`, `segments` (not in the reference either): the index made by `build_checkpoints`; the
    segments of every stream are then decoded side by side -- same bytes out, a shorter chain of steps."""
    K, N = int(output_shape[0]), int(output_shape[1])
    num_tiles_n, num_tiles_k = _tiles(K, N, tile_k, tile_n)
    _lib.require_device(compressed_streams)
    # comp_inference/rans_triton.py:141-144, extended to the other per-tile operands
    _lib.check_tiled_operands(K, N, int(tile_k), int(tile_n), initial_states, tables, slot_map, tile_offsets,
                              tile_max_lens, False)
    dev = compressed_streams.device
    stream_t = _lib.as_u8(compressed_streams, dev)
    merge = mantissas is not None
    if merge:
        man = _lib.as_u8(mantissas, dev).view(-1)
        need = num_tiles_k * num_tiles_n * tile_k * tile_n
        if man.numel() < need:  # a truncated tail reads as zero padding (comp_inference.py:76-83)
            man = torch.nn.functional.pad(man, (0, need - man.numel()))
    else:
        man = None
    want = torch.bfloat16 if merge else torch.uint8
    if out is None:
        out = torch.empty((K, N), device=dev, dtype=want)
    elif out.dtype != want or tuple(out.shape) != (K, N) or out.device != dev or not out.is_contiguous():
        raise RuntimeError(f"out must be a contiguous {want} tensor of shape ({K}, {N}) on {dev}")
    # device copies must stay referenced until the launch has been enqueued
    st, tb, sm = _lib.as_u32(initial_states, dev), _lib.as_u32(tables, dev), _lib.as_u8(slot_map, dev)
    to, tl = _lib.as_u32(tile_offsets, dev), _lib.as_u32(tile_max_lens, dev)
    ck, segments = _checked_checkpoints(checkpoints, segments, K, N, tile_k, tile_n, dev)
    # the lengths of every operand travel with it and are checked by the library before the launch
    w = _lib.tiled_weight(K, N, tile_k, tile_n, stream_t, st, tb, sm, to, tl, man, ck, segments)
    check(lib().ci_decode_tiled(C.byref(w), None if merge else ptr(out), ptr(out) if merge else None,
                                _lib.stream_handle(dev)))
    return out


def suggest_segments(weight_shape, tile_k=1024, tile_n=32) -> int:
    """Segments per stream (1, 2, 4 or 8) with which a weight of this shape fills the chip in the fused
    linear: 1 for weights with enough tiles of their own.  See `build_checkpoints`."""
    K, N = int(weight_shape[0]), int(weight_shape[1])
    return int(lib().ci_suggest_segments(K, N, int(tile_k), int(tile_n)))


def build_checkpoints(compressed_streams, initial_states, tables, slot_map, weight_shape, tile_offsets,
                      tile_max_lens, tile_k=1024, tile_n=32, segments=4):
    """Decoder checkpoints of a tiled-format tensor: state and byte position of every stream at `segments`
    evenly spaced rows, as an int64 tensor [tiles, segments - 1, 2 * tile_n] (low half state, high half
    row of the next unread byte), or None for segments <= 1.  An index kept beside the compressed
    tensor -- the stream is not changed -- which lets `fused_rans_linear(..., checkpoints=, segments=)`
    decode the segments of a stream at the same time instead of one after the other.  Not in the
    reference, whose tiled format has no checkpoints."""
    if segments <= 1:
        return None
    K, N = int(weight_shape[0]), int(weight_shape[1])
    _lib.require_device(compressed_streams)
    dev = compressed_streams.device
    tiles_n, tiles_k = _tiles(K, N, tile_k, tile_n)
    out = torch.empty((tiles_k * tiles_n, segments - 1, 2 * tile_n), dtype=torch.int64, device=dev)
    stream_t = _lib.as_u8(compressed_streams, dev)
    st, tb, sm = _lib.as_u32(initial_states, dev), _lib.as_u32(tables, dev), _lib.as_u8(slot_map, dev)
    to, tl = _lib.as_u32(tile_offsets, dev), _lib.as_u32(tile_max_lens, dev)
    check(lib().ci_build_checkpoints_ilp2(
        ptr(stream_t), C.c_uint64(stream_t.numel()), ptr(st), ptr(tb), ptr(sm), ptr(to), ptr(tl), K, N,
        int(tile_k), int(tile_n), int(segments), ptr(out), C.c_size_t(out.numel() * 8), _lib.stream_handle(dev)))
    return out


def build_slot_table(tables, slot_map, device=None) -> torch.Tensor:
    """The decoder's lookup table in the form the kernels keep in LDS (32 KB, uint8 tensor on the GPU): one
    8-byte entry per 12-bit slot, the reference's `slot_map` and `tables` folded into one read
    (src/cuda/rans_kernels.cuh:677-690).  Derived data kept beside a weight like the checkpoints: an operator
    given it copies the table instead of building it in every workgroup."""
    dev = torch.device(device) if device is not None else tables.device
    tb, sm = _lib.as_u32(tables, dev), _lib.as_u8(slot_map, dev)
    _lib.require_device(tb)
    if tb.numel() != 256 or sm.numel() != 4096:
        raise ValueError("tables must hold 256 entries and slot_map 4096")
    out = torch.empty(_lib.SLOT_TABLE_BYTES, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        check(lib().ci_build_slot_table(ptr(tb), ptr(sm), ptr(out), C.c_size_t(_lib.SLOT_TABLE_BYTES),
                                        _lib.stream_handle(dev)))
    return out


class _DecodeItem(C.Structure):
    _fields_ = [("d_stream", C.c_void_p), ("stream_len", C.c_uint64), ("d_states", C.c_void_p),
                ("d_tables", C.c_void_p), ("d_slot_map", C.c_void_p), ("d_tile_offsets", C.c_void_p),
                ("d_tile_max_lens", C.c_void_p), ("K", C.c_uint32), ("N", C.c_uint32),
                ("tile_height", C.c_uint32), ("tile_width", C.c_uint32), ("d_out_exp", C.c_void_p),
                ("d_checkpoints", C.c_void_p), ("segments", C.c_uint32)]


def rans_decomp_tiled_batch(items, tile_k=1024, tile_n=32):
    """Decode several tensors with one launch.  `items` is a sequence of tuples
    (compressed_streams, initial_states, tables, slot_map, output_shape, tile_offsets, tile_max_lens)
    -- the positional arguments of rans_decomp_tiled, optionally followed by (checkpoints, segments) --
    all on the same GPU; returns the list of exponent planes.  A stand-alone decode takes tile_k / 2
    dependent steps per wavefront whatever the tensor's size, so decoding a layer's tensors together
    keeps the whole chip busy."""
    items = list(items)
    if not items:
        return []
    _lib.require_device(items[0][0])
    dev = items[0][0].device
    arr = (_DecodeItem * len(items))()
    keep, outs = [], []
    for i, item in enumerate(items):
        cs, st, tb, sm, shape, to, tl = item[:7]
        K, N = int(shape[0]), int(shape[1])
        ck, segs = _checked_checkpoints(*(item[7:9] if len(item) >= 9 else (None, 1)), K, N, tile_k, tile_n, dev)
        _lib.check_tiled_operands(K, N, int(tile_k), int(tile_n), st, tb, sm, to, tl, False)
        t = (_lib.as_u8(cs, dev), _lib.as_u32(st, dev), _lib.as_u32(tb, dev), _lib.as_u8(sm, dev),
             _lib.as_u32(to, dev), _lib.as_u32(tl, dev))
        out = torch.empty((K, N), device=dev, dtype=torch.uint8)
        keep.append((t, ck))
        outs.append(out)
        arr[i] = _DecodeItem(t[0].data_ptr() if t[0].numel() else None, t[0].numel(), t[1].data_ptr(),
                             t[2].data_ptr(), t[3].data_ptr(), t[4].data_ptr(), t[5].data_ptr(), K, N,
                             int(tile_k), int(tile_n), out.data_ptr(), None if ck is None else ck.data_ptr(), segs)
    check(lib().ci_decode_tiled_ilp2_batch(arr, len(items), _lib.stream_handle(dev)))
    return outs


def rans_decomp_flat(compressed_streams, initial_states, tables, slot_map, stream_sizes, output_shape):
    """Decode the flat format (512-row segments per column) into u8[K,N]
    (comp_inference/rans_triton.py:243-271)."""
    _lib.require_device(compressed_streams)
    dev = compressed_streams.device
    K, N = int(output_shape[0]), int(output_shape[1])
    num_streams = len(initial_states)
    if stream_sizes.numel() != num_streams or tables.numel() != 256 or slot_map.numel() != 4096:
        raise ValueError(f"stream_sizes must hold {num_streams} entries, tables 256, slot_map 4096")
    out = torch.empty((K, N), device=dev, dtype=torch.uint8)
    stream_t = _lib.as_u8(compressed_streams, dev)
    st, sz = _lib.as_u32(initial_states, dev), _lib.as_u32(stream_sizes, dev)
    tb, sm = _lib.as_u32(tables, dev), _lib.as_u8(slot_map, dev)
    check(lib().ci_decode_flat_segmented(
        ptr(stream_t), C.c_uint64(stream_t.numel()), ptr(st), ptr(sz), num_streams, ptr(tb), ptr(sm), K, N, ptr(out), _lib.stream_handle(dev)))
    return out


def rans_decomp_tiled_uncoalesced(compressed_streams, initial_states, tables, slot_map, output_shape,
                                  stream_offsets, stream_sizes, tile_k=1024, tile_n=32, mantissas=None):
    """Decode the dense one-stream-per-column tiled format into u8[K,N] (or bf16 with
    `mantissas`).  The reference only decodes this layout inside its fused kernels
    (comp_inference/linear_triton.py:1045-1186); this op exists for round-trip checks."""
    _lib.require_device(compressed_streams)
    dev = compressed_streams.device
    K, N = int(output_shape[0]), int(output_shape[1])
    _lib.check_tiled_operands(K, N, int(tile_k), int(tile_n), initial_states, tables, slot_map, stream_offsets,
                              stream_sizes, True)
    stream_t = _lib.as_u8(compressed_streams, dev)
    merge = mantissas is not None
    man = None
    if merge:
        man = _lib.as_u8(mantissas, dev).view(-1)
        num_tiles_n, num_tiles_k = _tiles(K, N, tile_k, tile_n)
        need = num_tiles_k * num_tiles_n * tile_k * tile_n
        if man.numel() < need:  # a truncated tail reads as zero padding, as in rans_decomp_tiled
            man = torch.nn.functional.pad(man, (0, need - man.numel()))
    out = torch.empty((K, N), device=dev, dtype=torch.bfloat16 if merge else torch.uint8)
    st, tb, sm = _lib.as_u32(initial_states, dev), _lib.as_u32(tables, dev), _lib.as_u8(slot_map, dev)
    so, sz = _lib.as_u32(stream_offsets, dev), _lib.as_u32(stream_sizes, dev)
    check(lib().ci_decode_tiled_dense(
        ptr(stream_t), C.c_uint64(stream_t.numel()), ptr(st), ptr(tb), ptr(sm), ptr(so), ptr(sz),
        K, N, int(tile_k), int(tile_n), None if merge else ptr(out), ptr(man) if merge else None,
        ptr(out) if merge else None, _lib.stream_handle(dev)))
    return out


def rans_decomp_tiled_one_stream(compressed_streams, initial_states, tables, slot_map, output_shape,
                                 tile_offsets, tile_max_lens, tile_k=1024, tile_n=32, mantissas=None):
    """Decode the first tiled format -- one stream per column and tile, tile bodies of `tile_n` bytes a row --
    into u8[K,N] (`rans_decomp_triton_tiled_splitk`, comp_inference/rans_triton.py:468-516, and
    `rans_decomp_triton_tiled2`, :355-395, which runs the same kernel: the second definition at :399
    replaces the first of that name at :275), or into the bf16 weight with `mantissas`."""
    _lib.require_device(compressed_streams)
    dev = compressed_streams.device
    K, N = int(output_shape[0]), int(output_shape[1])
    # comp_inference/rans_triton.py:482-487, extended to the other per-tile operands
    _lib.check_tiled_operands(K, N, int(tile_k), int(tile_n), initial_states, tables, slot_map, tile_offsets,
                              tile_max_lens, False, True)
    stream_t = _lib.as_u8(compressed_streams, dev)
    merge = mantissas is not None
    man = None
    if merge:
        man = _lib.as_u8(mantissas, dev).view(-1)
        num_tiles_n, num_tiles_k = _tiles(K, N, tile_k, tile_n)
        need = num_tiles_k * num_tiles_n * tile_k * tile_n
        if man.numel() < need:  # a truncated tail reads as zero padding, as in rans_decomp_tiled
            man = torch.nn.functional.pad(man, (0, need - man.numel()))
    out = torch.empty((K, N), device=dev, dtype=torch.bfloat16 if merge else torch.uint8)
    st, tb, sm = _lib.as_u32(initial_states, dev), _lib.as_u32(tables, dev), _lib.as_u8(slot_map, dev)
    to, tl = _lib.as_u32(tile_offsets, dev), _lib.as_u32(tile_max_lens, dev)
    check(lib().ci_decode_tiled_one(
        ptr(stream_t), C.c_uint64(stream_t.numel()), ptr(st), ptr(tb), ptr(sm), ptr(to), ptr(tl),
        K, N, int(tile_k), int(tile_n), None if merge else ptr(out), ptr(man) if merge else None,
        ptr(out) if merge else None, _lib.stream_handle(dev)))
    return out


# Names under which the reference exports these ops (comp_inference/__init__.py:34-37).
rans_decomp_triton_tiled = rans_decomp_tiled
rans_decomp_triton = rans_decomp_flat
# (defined in comp_inference/rans_triton.py, not exported by the reference's package)
rans_decomp_triton_tiled_splitk = rans_decomp_tiled_one_stream
rans_decomp_triton_tiled2 = rans_decomp_tiled_one_stream
