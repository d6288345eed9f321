"""Fused decompress + linear against a row-per-output weight (LM head sharing the embedding
table's layout).  Call signatures follow comp_inference/transposed_linear_triton.py:361-377
(`fused_rans_linear_transposed_triton`) and :813-829 (`..._uncoalesced`); the kernels are HIP
(csrc/transposed.hip).
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from ._lib import check, lib, ptr
from . import linear_hip
from .linear_hip import _Scratch, _prep_x

# Rows of x above which the weight is decoded once into a bf16 scratch and multiplied with a library
# GEMM; the fused kernel walks the whole table once per 4 rows (128256 x 4096 table: 1286 us fused against
# 791 us at 5 rows, 23 ms against 0.83 ms at 128).  None switches the policy off.
DECODE_ONCE_ABOVE_ROWS = 4


def head_matrix_sums(enable: bool) -> bool:
    """One row of x on a weight with decoder checkpoints (the sixteen-wavefront kernel): with `enable` the sums over
    the hidden dimension are formed on the matrix pipe instead of by lane exchanges -- fewer vector instructions per
    symbol, another order of the sum (same tolerance, not bit-identical to the other kernels), finite weights only
    (0 x Inf = NaN would spoil the other rows of a group of 32).  Process-wide, off by default; returns the previous
    setting."""
    return bool(lib().ci_fused_linear_transposed_matrix_sums(1 if enable else 0))


def _run(x, compressed_data, initial_states, tables, slot_map, weight_shape, meta0, meta1, tile_k, tile_n,
         mantissas, bias, out, dense: bool, checkpoints=None, segments: int = 1, max_window_rows: int = 0,
         slot_table=None, one: bool = False):
    V, H = int(weight_shape[0]), int(weight_shape[1])  # weight is [vocab, hidden]
    _lib.require_device(x)
    _lib.check_tiled_operands(V, H, int(tile_k), int(tile_n), initial_states, tables, slot_map, meta0, meta1, dense, one)
    dev = x.device
    x2 = _prep_x(x, H)
    M = x2.shape[0]
    if out is None:
        result = torch.empty((M, V), dtype=torch.bfloat16, device=dev)
    else:
        if out.dtype != torch.bfloat16 or not out.is_cuda:
            raise RuntimeError("out must be a bfloat16 GPU tensor")
        result = out.view(M, V)
    if not dense and not one and DECODE_ONCE_ABOVE_ROWS is not None and M > DECODE_ONCE_ABOVE_ROWS:
        w = linear_hip._decode_once_weight(dev, compressed_data, initial_states, tables, slot_map, (V, H), meta0, meta1,
                                           int(tile_k), int(tile_n), mantissas, "weight_vh")
        if result.is_contiguous():
            torch.matmul(x2.detach(), w.t(), out=result)  # (like the fused kernels: inference only)
        else:
            result.copy_(torch.matmul(x2.detach(), w.t()))
        if bias is not None:
            result += bias.to(device=dev, dtype=torch.bfloat16)
        return out if out is not None else result.view(*x.shape[:-1], V)
    stream_t = _lib.as_u8(compressed_data, dev)
    man = _lib.as_u8(mantissas, dev).view(-1)
    need_man = (-(-V // tile_k)) * (-(-H // tile_n)) * tile_k * tile_n
    if man.numel() < need_man:
        man = torch.nn.functional.pad(man, (0, need_man - man.numel()))
    need = lib().ci_fused_linear_transposed_workspace_bytes(M, H, V, int(tile_n))
    ws = _Scratch.get(need, ("lmhead", dev))
    b = bias.to(device=dev, dtype=torch.bfloat16).contiguous() if bias is not None else None
    # device copies must stay referenced until the launch has been enqueued
    st, tb, sm = _lib.as_u32(initial_states, dev), _lib.as_u32(tables, dev), _lib.as_u8(slot_map, dev)
    m0, m1 = _lib.as_u32(meta0, dev), _lib.as_u32(meta1, dev)
    if dense or one:
        entry = lib().ci_fused_linear_transposed_one if one else lib().ci_fused_linear_transposed_dense
        check(entry(
            ptr(x2), M, H, V, x2.stride(0), ptr(stream_t), C.c_uint64(stream_t.numel()), ptr(st), ptr(tb), ptr(sm),
            ptr(m0), ptr(m1), ptr(man), int(tile_k), int(tile_n), ptr(b), ptr(result), result.stride(0), ptr(ws),
            C.c_size_t(ws.numel()), _lib.stream_handle(dev)))
    else:
        # the lengths of every operand travel with it and are checked by the library before the launch
        ck = None
        if checkpoints is not None and int(segments) > 1:
            ck = checkpoints.to(dev).contiguous()
            if ck.dtype != torch.int64:
                raise RuntimeError("checkpoints do not belong to this weight shape, tiling and segment count")
        w = _lib.tiled_weight(V, H, tile_k, tile_n, stream_t, st, tb, sm, m0, m1, man, ck, int(segments) if ck is not None else 1,
                              slot_table, int(max_window_rows))
        check(lib().ci_fused_linear_transposed_tiled(C.byref(w), ptr(x2), M, x2.stride(0), ptr(b), ptr(result),
                                                     result.stride(0), ptr(ws), C.c_size_t(ws.numel()),
                                                     _lib.stream_handle(dev)))
    if out is not None:
        return out
    return result.view(*x.shape[:-1], V)


def fused_rans_linear_transposed(x, compressed_data, initial_states, tables, slot_map, weight_shape,
                                 tile_offsets, tile_max_lens, tile_k, tile_n, mantissas, workspace=None,
                                 bias=None, out=None, SPLIT_K=8, checkpoints=None, segments=1, max_window_rows=0,
                                 slot_table=None):
    """x[..., H] @ W[V, H]^T (+ bias), W in the tiled two-streams-per-column format
    (comp_inference/transposed_linear_triton.py:361-435).  `workspace` and `SPLIT_K` are accepted
    for signature compatibility; the library keeps its own fp32 scratch (one partial per column
    tile, summed in tile order)."""
    return _run(x, compressed_data, initial_states, tables, slot_map, weight_shape, tile_offsets, tile_max_lens,
                tile_k, tile_n, mantissas, bias, out, dense=False, checkpoints=checkpoints, segments=segments,
                max_window_rows=max_window_rows, slot_table=slot_table)


def fused_rans_linear_transposed_uncoalesced(x, compressed_data, initial_states, tables, slot_map, weight_shape,
                                             stream_offsets, stream_sizes, tile_k, tile_n, mantissas,
                                             workspace=None, bias=None, out=None, SPLIT_K=8):
    """Same for the dense one-stream-per-column layout
    (comp_inference/transposed_linear_triton.py:813-883)."""
    return _run(x, compressed_data, initial_states, tables, slot_map, weight_shape, stream_offsets, stream_sizes,
                tile_k, tile_n, mantissas, bias, out, dense=True)


def fused_rans_linear_transposed_one_stream(x, compressed_data, initial_states, tables, slot_map, weight_shape,
                                            tile_offsets, tile_max_lens, tile_k, tile_n, mantissas, bias=None, out=None):
    """Same for the first tiled format, one stream per column and tile in tile bodies of `tile_n` bytes a row:
    what `fused_rans_linear_transposed_triton_2` (comp_inference/transposed_linear_triton.py:438-500) is
    written for.  The reference's function cannot run -- the kernel it launches,
    `fused_rans_matmul_transposed_kernel` (:469), is defined nowhere -- so the result is pinned by the
    decoded weight and a matmul, not by that function."""
    return _run(x, compressed_data, initial_states, tables, slot_map, weight_shape, tile_offsets, tile_max_lens,
                tile_k, tile_n, mantissas, bias, out, dense=False, one=True)


def plain_linear_transposed_same_order(x, weight_vh, tile_k=1024, tile_n=32, bias=None):
    """x[..., H] @ weight_vh[V, H]^T (+ bias) for an uncompressed bf16 weight, through the fused
    kernel's own products and reductions: bit-identical to `fused_rans_linear_transposed` on the
    compressed form of `weight_vh` (tile `tile_k` x 32).  A verification aid without a counterpart in
    the reference; slow."""
    _lib.require_device(x)
    _lib.require_device(weight_vh)
    if weight_vh.dtype != torch.bfloat16 or weight_vh.dim() != 2:
        raise RuntimeError("weight_vh must be a 2-D bfloat16 tensor [V, H]")
    dev = x.device
    w = weight_vh.contiguous()
    V, H = w.shape
    x2 = _prep_x(x, H)
    M = x2.shape[0]
    if DECODE_ONCE_ABOVE_ROWS is not None and M > DECODE_ONCE_ABOVE_ROWS:
        # what fused_rans_linear_transposed computes for this many rows: a library GEMM on the decoded weight
        result = torch.matmul(x2, w.t())
        if bias is not None:
            result += bias.to(device=dev, dtype=torch.bfloat16)
        return result.view(*x.shape[:-1], V)
    result = torch.empty((M, V), dtype=torch.bfloat16, device=dev)
    need = lib().ci_fused_linear_transposed_workspace_bytes(M, H, V, int(tile_n))
    ws = _Scratch.get(need, ("lmhead", dev))
    b = bias.to(device=dev, dtype=torch.bfloat16).contiguous() if bias is not None else None
    check(lib().ci_plain_linear_transposed_same_order(ptr(x2), M, H, V, x2.stride(0), ptr(w), int(tile_k), int(tile_n),
                                                      ptr(b), ptr(result), result.stride(0), ptr(ws),
                                                      C.c_size_t(ws.numel()), _lib.stream_handle(dev)))
    return result.view(*x.shape[:-1], V)


# Names under which the reference exports these ops (comp_inference/__init__.py:44-47).
fused_rans_linear_transposed_triton = fused_rans_linear_transposed
fused_rans_linear_transposed_triton_uncoalesced = fused_rans_linear_transposed_uncoalesced
fused_rans_linear_transposed_triton_2 = fused_rans_linear_transposed_one_stream  # (defined there, not exported)
