"""Fused decompress + embedding gather on the GPU.

Call signatures follow comp_inference/embedding_triton.py:278-291 (`fused_rans_embedding_triton`),
:431-444 (`fused_rans_embedding_triton_uncoalesced`) and :8-21 (`fused_rans_embedding_triton_2`); the kernels are HIP (csrc/embedding.hip).
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from ._lib import check, lib, ptr
from .linear_hip import _Scratch


def _run(x, compressed_data, initial_states, tables, slot_map, weight_shape, meta0, meta1, tile_k, tile_n,
         mantissas, out, dense: bool, checkpoints=None, segments: int = 1, one: bool = False, slot_table=None):
    K, N = int(weight_shape[0]), int(weight_shape[1])  # K = vocabulary, N = hidden
    _lib.require_device(x)
    _lib.check_tiled_operands(K, N, int(tile_k), int(tile_n), initial_states, tables, slot_map, meta0, meta1, dense, one)
    dev = x.device
    ids = x.reshape(-1)
    if ids.dtype != torch.int64:
        ids = ids.to(torch.int64)
    ids = ids.contiguous()
    n = ids.numel()
    if out is None:
        result = torch.empty((n, N), device=dev, dtype=torch.bfloat16)
    else:
        if out.dtype != torch.bfloat16 or not out.is_cuda:
            raise RuntimeError("out must be a bfloat16 GPU tensor")
        result = out.view(n, N)
    stream_t = _lib.as_u8(compressed_data, dev)
    man = _lib.as_u8(mantissas, dev).view(-1)
    need_man = (-(-K // tile_k)) * (-(-N // tile_n)) * tile_k * tile_n
    if man.numel() < need_man:
        man = torch.nn.functional.pad(man, (0, need_man - man.numel()))
    # device copies must stay referenced until the launch has been enqueued
    st, tb, sm = _lib.as_u32(initial_states, dev), _lib.as_u32(tables, dev), _lib.as_u8(slot_map, dev)
    m0, m1 = _lib.as_u32(meta0, dev), _lib.as_u32(meta1, dev)
    if dense or one:
        entry = lib().ci_fused_embedding_one if one else lib().ci_fused_embedding_dense
        check(entry(
            ptr(ids), n, ptr(stream_t), C.c_uint64(stream_t.numel()), ptr(st), ptr(tb), ptr(sm), ptr(m0), ptr(m1),
            ptr(man), K, N, int(tile_k), int(tile_n), ptr(result), result.stride(0), _lib.stream_handle(dev)))
    else:
        ck, segments = None, 1 if checkpoints is None else int(segments)
        if segments > 1:
            ck = checkpoints.to(dev).contiguous()
            if ck.dtype != torch.int64:
                raise RuntimeError("checkpoints do not belong to this table shape, tiling and segment count")
        need = lib().ci_fused_embedding_workspace_bytes_segmented(n, K, int(tile_k), segments)
        ws = _Scratch.get(need, ("emb", dev))
        # the lengths of every operand travel with it and are checked by the library before the launch
        w = _lib.tiled_weight(K, N, tile_k, tile_n, stream_t, st, tb, sm, m0, m1, man, ck, segments, slot_table)
        check(lib().ci_fused_embedding_tiled(C.byref(w), ptr(ids), n, ptr(result), result.stride(0), ptr(ws),
                                             C.c_size_t(ws.numel() if ws is not None else 0), _lib.stream_handle(dev)))
    if out is not None:
        return out.view(*x.shape, N)
    return result.view(*x.shape, N)


def fused_rans_embedding(x, compressed_data, initial_states, tables, slot_map, weight_shape, tile_offsets,
                         tile_max_lens, tile_k, tile_n, mantissas, out=None, checkpoints=None, segments=1,
                         slot_table=None):
    """table[x] for a table in the tiled two-streams-per-column format; ids outside the table give
    zero rows (comp_inference/embedding_triton.py:204-210, :278-330).  `checkpoints`, `segments` (not in
    the reference): the index made by `rans_hip.build_checkpoints`; a row then costs at most
    tile_k / (2 segments) decode steps instead of tile_k / 2.  `slot_table` (not in the reference):
    the table made by `rans_hip.build_slot_table`; with it and checkpoints that cut buckets of at most 128 rows
    the gather runs on sixteen wavefronts per CU with every load of an item asked for ahead of it."""
    return _run(x, compressed_data, initial_states, tables, slot_map, weight_shape, tile_offsets, tile_max_lens,
                tile_k, tile_n, mantissas, out, dense=False, checkpoints=checkpoints, segments=segments,
                slot_table=slot_table)


def fused_rans_embedding_uncoalesced(x, compressed_data, initial_states, tables, slot_map, weight_shape,
                                     stream_offsets, stream_sizes, tile_k, tile_n, mantissas, out=None):
    """Same for the dense one-stream-per-column layout (comp_inference/embedding_triton.py:431-483)."""
    return _run(x, compressed_data, initial_states, tables, slot_map, weight_shape, stream_offsets, stream_sizes,
                tile_k, tile_n, mantissas, out, dense=True)


def fused_rans_embedding_one_stream(x, compressed_data, initial_states, tables, slot_map, weight_shape,
                                    tile_offsets, tile_max_lens, tile_k, tile_n, mantissas, out=None):
    """Same for the first tiled format, one stream per column and tile in tile bodies of `tile_n` bytes a row
    (`fused_rans_embedding_triton_2`, comp_inference/embedding_triton.py:8-67; kernel :71-167)."""
    return _run(x, compressed_data, initial_states, tables, slot_map, weight_shape, tile_offsets, tile_max_lens,
                tile_k, tile_n, mantissas, out, dense=False, one=True)


# Names under which the reference exports these ops (comp_inference/__init__.py:49-52).
fused_rans_embedding_triton = fused_rans_embedding
fused_rans_embedding_triton_uncoalesced = fused_rans_embedding_uncoalesced
fused_rans_embedding_triton_2 = fused_rans_embedding_one_stream  # (defined there, not exported by the reference)
