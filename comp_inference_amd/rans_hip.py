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


def rans_decomp_tiled(compressed_streams, initial_states, tables, slot_map, output_shape,
                      tile_offsets, tile_max_lens, tile_k=1024, tile_n=32, mantissas=None):
    """Decode the tiled two-streams-per-column format into the exponent plane u8[K,N]
    (comp_inference/rans_triton.py:122-168).  With `mantissas` (the tile-interleaved sign|mantissa
    plane) the bf16 weight [K,N] is returned instead, merged in the same kernel."""
    K, N = int(output_shape[0]), int(output_shape[1])
    num_tiles_n, num_tiles_k = _tiles(K, N, tile_k, tile_n)
    expected_streams = num_tiles_n * num_tiles_k * tile_n * 2
    if initial_states.numel() != expected_streams:
        # comp_inference/rans_triton.py:141-144
        raise ValueError(f"Initial states size mismatch. Expected {expected_streams}")
    _lib.require_device(compressed_streams)
    dev = compressed_streams.device
    stream_t = _lib.as_u8(compressed_streams, dev)
    merge = mantissas is not None
    if merge:
        man = _lib.as_u8(mantissas, dev).view(-1)
        need = num_tiles_k * num_tiles_n * tile_k * tile_n
        if man.numel() < need:  # a truncated tail reads as zero padding (comp_inference.py:76-83)
            man = torch.nn.functional.pad(man, (0, need - man.numel()))
        out = torch.empty((K, N), device=dev, dtype=torch.bfloat16)
    else:
        man = None
        out = torch.empty((K, N), device=dev, dtype=torch.uint8)
    # device copies must stay referenced until the launch has been enqueued
    st, tb, sm = _lib.as_u32(initial_states, dev), _lib.as_u32(tables, dev), _lib.as_u8(slot_map, dev)
    to, tl = _lib.as_u32(tile_offsets, dev), _lib.as_u32(tile_max_lens, dev)
    check(lib().ci_decode_tiled_ilp2(
        ptr(stream_t), C.c_uint64(stream_t.numel()), ptr(st), ptr(tb), ptr(sm), ptr(to), ptr(tl),
        K, N, int(tile_k), int(tile_n), None if merge else ptr(out), ptr(man) if merge else None,
        ptr(out) if merge else None, _lib.stream_handle(dev)))
    return out


def rans_decomp_flat(compressed_streams, initial_states, tables, slot_map, stream_sizes, output_shape):
    """Decode the flat format (512-row segments per column) into u8[K,N]
    (comp_inference/rans_triton.py:243-271)."""
    _lib.require_device(compressed_streams)
    dev = compressed_streams.device
    K, N = int(output_shape[0]), int(output_shape[1])
    num_streams = len(initial_states)
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
    stream_t = _lib.as_u8(compressed_streams, dev)
    merge = mantissas is not None
    man = _lib.as_u8(mantissas, dev).view(-1) if merge else None
    out = torch.empty((K, N), device=dev, dtype=torch.bfloat16 if merge else torch.uint8)
    st, tb, sm = _lib.as_u32(initial_states, dev), _lib.as_u32(tables, dev), _lib.as_u8(slot_map, dev)
    so, sz = _lib.as_u32(stream_offsets, dev), _lib.as_u32(stream_sizes, dev)
    check(lib().ci_decode_tiled_dense(
        ptr(stream_t), C.c_uint64(stream_t.numel()), ptr(st), ptr(tb), ptr(sm), ptr(so), ptr(sz),
        K, N, int(tile_k), int(tile_n), None if merge else ptr(out), ptr(man) if merge else None,
        ptr(out) if merge else None, _lib.stream_handle(dev)))
    return out


# Names under which the reference exports these ops (comp_inference/__init__.py:34-37).
rans_decomp_triton_tiled = rans_decomp_tiled
rans_decomp_triton = rans_decomp_flat
