"""Fused decompress + linear on the GPU.

Call signatures follow comp_inference/linear_triton.py:229-246 (`fused_rans_linear_triton`) and
:1189-1206 (`fused_rans_linear_triton_uncoalesced`).  The kernels are HIP (csrc/linear.hip): the
weight is decoded tile by tile inside the GEMV/GEMM and never written to memory.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from ._lib import check, lib, ptr, stream_handle


class _Scratch:
    """Scratch areas (split-K partials, decoded weights, sort keys), one per purpose, device and stream (the
    reference keeps a class-level buffer too, comp_inference/pytorch_runtime.py:386-394).  Calls that follow
    each other on one stream share an area safely; calls on different streams get areas of their own.  An
    area grows to the largest request it has seen and stays: the decode-once path of a many-row linear keeps
    one bf16 weight (117 MB for a 4096 x 14336 projection, 1 GB for a 128256 x 4096 head) until
    `release_scratch()` is called or `DECODE_ONCE_ABOVE_ROWS` is set to None."""
    _buf: dict = {}

    @classmethod
    def get(cls, nbytes: int, key) -> torch.Tensor | None:
        """`key` is a device, or a (tag, device) pair for a scratch area of its own."""
        if nbytes == 0:
            return None
        device = key[1] if isinstance(key, tuple) else key
        key = (key, torch.cuda.current_stream(device).cuda_stream)
        b = cls._buf.get(key)
        if b is None or b.numel() < nbytes:
            b = torch.empty(nbytes, dtype=torch.uint8, device=device)
            cls._buf[key] = b
        return b

    @classmethod
    def release(cls) -> int:
        """Drops every scratch area; returns the bytes given back to torch's allocator."""
        n = sum(b.numel() for b in cls._buf.values())
        cls._buf.clear()
        return n


def release_scratch() -> int:
    """Frees the scratch areas the operators keep between calls (they are allocated again on demand).  Not
    while a captured graph that uses them may still be replayed."""
    return _Scratch.release()


# Rows of x above which the fused linear decodes the weight ONCE into a bf16 scratch and multiplies with
# a library GEMM (hipBLASLt through torch.matmul), instead of decoding it inside the product once per
# 64 rows: with hundreds of prompt tokens the decode, not the product, would otherwise be repeated
# (gate projection 4096 x 14336: 121 us fused against 96 us at 96 rows, 1497 against 264 at 2048).
# None switches the policy off.  The reference always fuses, one decode per 16 rows
# (comp_inference/linear_triton.py:250-266).
DECODE_ONCE_ABOVE_ROWS = 64


def fused_wide_rows(enable: bool) -> bool:
    """More than 64 rows of x inside the fused kernel (reached with DECODE_ONCE_ABOVE_ROWS = None, or from C):
    with `enable` a tile is decoded once per 128 or 256 rows of x instead of once per 64.  Bit-identical results.
    Process-wide, off by default; returns the previous setting."""
    return bool(lib().ci_fused_linear_wide_rows(1 if enable else 0))


def device_status(device=None) -> int:
    """What the kernels could not do and did not hang over since the last call, as CI_STATUS_* bits (0: nothing);
    raises RuntimeError if a bit is set.  Waits for the device's current stream: for health checks, not the token loop."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    word = C.c_uint32(0)
    with torch.cuda.device(dev):
        check(lib().ci_device_status(C.byref(word), stream_handle(dev)))
    return word.value


def debug_wait_limit(looks: int) -> int:
    """Looks a wavefront takes at another wavefront's flag before it gives up (ci_debug_wait_limit); returns the
    previous value.  0 forces the give-up path: for tests."""
    lib().ci_debug_wait_limit.restype = C.c_uint32
    return int(lib().ci_debug_wait_limit(C.c_uint32(int(looks))))


def _decode_once_weight(dev, compressed_data, initial_states, tables, slot_map, shape, tile_offsets, tile_max_lens,
                        tile_k, tile_n, mantissas, tag, checkpoints=None, segments=1):
    """The bf16 weight, decoded into a grow-only scratch of its own (valid until the next such call).  With
    the weight's decoder checkpoints the segments of a stream are decoded side by side (a 4096 x 4096
    weight: 53 -> 30 us)."""
    from .rans_hip import rans_decomp_tiled

    rows, cols = shape
    buf = _Scratch.get(rows * cols * 2, (tag, dev))
    w = buf[:rows * cols * 2].view(torch.bfloat16).view(rows, cols)
    return rans_decomp_tiled(compressed_data, initial_states, tables, slot_map, (rows, cols), tile_offsets,
                             tile_max_lens, tile_k=tile_k, tile_n=tile_n, mantissas=mantissas, out=w,
                             checkpoints=checkpoints, segments=segments)


def _prep_x(x: torch.Tensor, K: int):
    if x.dtype != torch.bfloat16:
        x = x.to(torch.bfloat16)  # the kernel computes on bf16 (comp_inference/linear_triton.py:431-436)
    x2 = x.reshape(-1, K)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    return x2


def _pick_workspace(workspace, need: int, dev):
    """A caller-supplied workspace is used when it is large enough for this library's fp32
    partials; the reference sizes it for its own bf16 partials, which may be smaller."""
    if need == 0:
        return None, 0
    if workspace is not None and workspace.is_cuda and workspace.is_contiguous() \
            and workspace.numel() * workspace.element_size() >= need:
        return workspace, workspace.numel() * workspace.element_size()
    buf = _Scratch.get(need, dev)
    return buf, buf.numel()


def _run(x, compressed_data, initial_states, tables, slot_map, weight_shape, meta0, meta1, tile_k,
         tile_n, mantissas, bias, out, workspace, dense: bool, checkpoints=None, segments: int = 1, one: bool = False):
    K, N = int(weight_shape[0]), int(weight_shape[1])
    _lib.require_device(x)
    _lib.check_tiled_operands(K, N, int(tile_k), int(tile_n), initial_states, tables, slot_map, meta0, meta1, dense, one)
    dev = x.device
    x2 = _prep_x(x, K)
    M = x2.shape[0]
    if out is None:
        result = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    else:
        if out.dtype != torch.bfloat16 or not out.is_cuda:
            raise RuntimeError("out must be a bfloat16 GPU tensor")
        result = out.view(M, N) if out.is_contiguous() else out
        if result.stride(-1) != 1:
            raise RuntimeError("out must have unit stride in its last dimension")
    if not dense and not one and DECODE_ONCE_ABOVE_ROWS is not None and M > DECODE_ONCE_ABOVE_ROWS:
        w = _decode_once_weight(dev, compressed_data, initial_states, tables, slot_map, (K, N), meta0, meta1,
                                int(tile_k), int(tile_n), mantissas, "weight_kn", checkpoints, segments)
        if result.is_contiguous():
            torch.matmul(x2.detach(), w, out=result)  # (like the fused kernels: inference only)
        else:
            result.copy_(torch.matmul(x2.detach(), w))
        if bias is not None:  # the reference's `out += bias` on the bf16 result
            result += bias.to(device=dev, dtype=torch.bfloat16)
        return out if out is not None else result.view(*x.shape[:-1], N)
    stream_t = _lib.as_u8(compressed_data, dev)
    man = _lib.as_u8(mantissas, dev).view(-1)
    need_man = (-(-K // tile_k)) * (-(-N // tile_n)) * tile_k * tile_n
    if man.numel() < need_man:
        man = torch.nn.functional.pad(man, (0, need_man - man.numel()))
    segments = int(segments) if checkpoints is not None and not dense and not one else 1
    need = lib().ci_fused_linear_workspace_bytes_segmented(M, K, N, int(tile_k), int(tile_n), int(dense or one), segments)
    ws, ws_bytes = _pick_workspace(workspace, need, dev)
    b = None
    if bias is not None:
        b = bias.to(device=dev, dtype=torch.bfloat16).contiguous()
    # device copies must stay referenced until the launch has been enqueued
    st, tb, sm = _lib.as_u32(initial_states, dev), _lib.as_u32(tables, dev), _lib.as_u8(slot_map, dev)
    m0, m1 = _lib.as_u32(meta0, dev), _lib.as_u32(meta1, dev)
    if not dense and not one:
        ck = None
        if segments > 1:
            ck = checkpoints.to(dev).contiguous()
            if ck.dtype != torch.int64:
                raise RuntimeError("checkpoints do not belong to this weight shape, tiling and segment count")
        # the lengths of every operand travel with it and are checked by the library before the launch
        w = _lib.tiled_weight(K, N, tile_k, tile_n, stream_t, st, tb, sm, m0, m1, man, ck, segments)
        check(lib().ci_fused_linear_tiled(C.byref(w), ptr(x2), M, x2.stride(0), ptr(b), ptr(result), result.stride(0),
                                          ptr(ws), C.c_size_t(ws_bytes), _lib.stream_handle(dev)))
    else:
        entry = lib().ci_fused_linear_one if one else lib().ci_fused_linear_dense
        check(entry(
            ptr(x2), M, K, N, x2.stride(0), ptr(stream_t), C.c_uint64(stream_t.numel()), ptr(st), ptr(tb), ptr(sm),
            ptr(m0), ptr(m1), ptr(man), int(tile_k), int(tile_n), ptr(b), ptr(result), result.stride(0), ptr(ws),
            C.c_size_t(ws_bytes), _lib.stream_handle(dev)))
    if out is not None:
        return out
    return result.view(*x.shape[:-1], N)


class PreparedLinear:
    """One compressed weight with everything a call needs converted once: device tensors, their
    pointers, the checkpoint index, the workspace size per row count.  `RansLinear` keeps one per device; a
    call then costs one output allocation and one library call instead of a dozen tensor conversions.
    Same kernels, same results as `fused_rans_linear`."""

    def __init__(self, dev, compressed_data, initial_states, tables, slot_map, weight_shape, tile_offsets,
                 tile_max_lens, tile_k, tile_n, mantissas, bias=None, checkpoints=None, segments=1):
        self.dev = dev
        self.K, self.N = int(weight_shape[0]), int(weight_shape[1])
        self.tile_k, self.tile_n = int(tile_k), int(tile_n)
        _lib.check_tiled_operands(self.K, self.N, self.tile_k, self.tile_n, initial_states, tables, slot_map,
                                  tile_offsets, tile_max_lens, False)
        man = _lib.as_u8(mantissas, dev).view(-1)
        need_man = (-(-self.K // self.tile_k)) * (-(-self.N // self.tile_n)) * self.tile_k * self.tile_n
        if man.numel() < need_man:
            man = torch.nn.functional.pad(man, (0, need_man - man.numel()))
        self.segments = int(segments) if checkpoints is not None else 1
        ck = None
        if self.segments > 1:
            ck = checkpoints.to(dev).contiguous()
            if ck.dtype != torch.int64 or \
                    ck.numel() * 8 != lib().ci_checkpoint_bytes(self.K, self.N, self.tile_k, self.tile_n, self.segments):
                raise RuntimeError("checkpoints do not belong to this weight shape, tiling and segment count")
        # the tensors stay referenced here for as long as their pointers are in use
        self.keep = (_lib.as_u8(compressed_data, dev), _lib.as_u32(initial_states, dev), _lib.as_u32(tables, dev),
                     _lib.as_u8(slot_map, dev), _lib.as_u32(tile_offsets, dev), _lib.as_u32(tile_max_lens, dev), man,
                     None if bias is None else bias.to(device=dev, dtype=torch.bfloat16).contiguous(), ck)
        # the decoder's lookup table in the form the kernels keep in LDS: built once, copied by every launch
        self.slot_table = torch.empty(_lib.SLOT_TABLE_BYTES, dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            check(lib().ci_build_slot_table(ptr(self.keep[2]), ptr(self.keep[3]), ptr(self.slot_table),
                                            C.c_size_t(_lib.SLOT_TABLE_BYTES), _lib.stream_handle(dev)))
        self.need = {}
        self.max_window_rows = 0
        self._bind()
        # the most rows of a tile body one item reads, worked out once (one small launch and a read-back): with
        # it in the descriptor the library knows that every item fits its staging area before it launches
        if self.tile_n == 32 and self.tile_k % 2 == 0 and (self.tile_k // 2) % self.segments == 0:
            rows = torch.zeros(1, dtype=torch.int32, device=dev)
            with torch.cuda.device(dev):
                check(lib().ci_max_window_rows(C.byref(self.w), ptr(rows), _lib.stream_handle(dev)))
            self.max_window_rows = int(rows.item())
            self._bind()

    def _bind(self) -> None:
        o = self.keep
        self.p = [ptr(t) for t in o]
        self.w = _lib.tiled_weight(self.K, self.N, self.tile_k, self.tile_n, o[0], o[1], o[2], o[3], o[4], o[5], o[6],
                                   o[8], self.segments, self.slot_table, self.max_window_rows)

    # A copy (copy.deepcopy of the owning module, pickling) gets its own tensors: the pointers are taken
    # again from them instead of travelling as numbers.
    def __getstate__(self):
        state = dict(self.__dict__)
        del state["p"], state["w"]
        return state

    def __setstate__(self, state):
        self.__dict__.update(state)
        self._bind()

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        if x.device != self.dev:
            raise RuntimeError(f"x is on {x.device}, the prepared weight on {self.dev}")
        x2 = _prep_x(x, self.K)
        M = x2.shape[0]
        if DECODE_ONCE_ABOVE_ROWS is not None and M > DECODE_ONCE_ABOVE_ROWS:
            o = self.keep
            return _run(x, o[0], o[1], o[2], o[3], (self.K, self.N), o[4], o[5], self.tile_k, self.tile_n, o[6],
                        o[7], None, None, dense=False, checkpoints=o[8], segments=self.segments)
        result = torch.empty((M, self.N), dtype=torch.bfloat16, device=self.dev)
        need = self.need.get(M)
        if need is None:
            need = self.need[M] = lib().ci_fused_linear_workspace_bytes_segmented(M, self.K, self.N, self.tile_k,
                                                                                   self.tile_n, 0, self.segments)
        ws, ws_bytes = _pick_workspace(None, need, self.dev)
        check(lib().ci_fused_linear_tiled(C.byref(self.w), ptr(x2), M, x2.stride(0), self.p[7], ptr(result), self.N,
                                          ptr(ws), C.c_size_t(ws_bytes), _lib.stream_handle(self.dev)))
        return result.view(*x.shape[:-1], self.N)


def fused_rans_linear(x, compressed_data, initial_states, tables, slot_map, weight_shape, tile_offsets,
                      tile_max_lens, tile_k, tile_n, mantissas, accum_block_size=32, bias=None, out=None,
                      SPLIT_K=8, workspace=None, checkpoints=None, segments=1):
    """x[..., K] @ W[K, N] (+ bias) with W in the tiled two-streams-per-column format
    (comp_inference/linear_triton.py:229-315).  `accum_block_size` and `SPLIT_K` are accepted for
    signature compatibility: the kernel always gives every tile its own wavefront and sums the
    per-tile partials in a fixed order, which is the finest split the format allows.
    `checkpoints`, `segments` (not in the reference): the index made by `build_checkpoints`, with which
    every segment of every tile gets a wavefront of its own -- for weights with few tiles."""
    return _run(x, compressed_data, initial_states, tables, slot_map, weight_shape, tile_offsets,
                tile_max_lens, tile_k, tile_n, mantissas, bias, out, workspace, dense=False,
                checkpoints=checkpoints, segments=segments)


def fused_rans_linear_uncoalesced(x, compressed_data, initial_states, tables, slot_map, weight_shape,
                                  stream_offsets, stream_sizes, tile_k, tile_n, mantissas,
                                  accum_block_size=32, bias=None, out=None, SPLIT_K=8, workspace=None):
    """Same for the dense one-stream-per-column layout (comp_inference/linear_triton.py:1189-1265)."""
    return _run(x, compressed_data, initial_states, tables, slot_map, weight_shape, stream_offsets,
                stream_sizes, tile_k, tile_n, mantissas, bias, out, workspace, dense=True)


def fused_rans_linear_one_stream(x, compressed_data, initial_states, tables, slot_map, weight_shape, tile_offsets,
                                 tile_max_lens, tile_k, tile_n, mantissas, accum_block_size=32, bias=None, out=None,
                                 SPLIT_K=8, workspace=None):
    """Same for the first tiled format, one stream per column and tile in tile bodies of `tile_n` bytes a row
    (`fused_rans_linear_triton_splitk`, comp_inference/linear_triton.py:806-890; kernel :893-1035).  The
    reference sums bf16 partials of SPLIT_K groups of tile rows with torch.sum; here every tile row has an
    fp32 partial of its own, summed in order and rounded once."""
    return _run(x, compressed_data, initial_states, tables, slot_map, weight_shape, tile_offsets,
                tile_max_lens, tile_k, tile_n, mantissas, bias, out, workspace, dense=False, one=True)


def fused_rans_linear_triton_2(x, compressed_data, initial_states, tables, slot_map, weight_shape, tile_offsets,
                               tile_max_lens, tile_k, tile_n, mantissas, accum_block_size=16, bias=None, out=None):
    """comp_inference/linear_triton.py:705-803: despite its name it launches the two-streams-per-column kernel
    (:769), so it is `fused_rans_linear` without the split-K arguments."""
    return fused_rans_linear(x, compressed_data, initial_states, tables, slot_map, weight_shape, tile_offsets,
                             tile_max_lens, tile_k, tile_n, mantissas, accum_block_size, bias, out)


def splitk_reduce(workspace: torch.Tensor, bias=None, out=None):
    """out = sum over dim 0 of a [SPLIT_K, M, N] workspace (+ bias), fp32 accumulate, one rounding
    to bf16: the reduction the reference performs with torch.sum
    (comp_inference/linear_triton.py:303-314).  Accepts bf16 or fp32 partials."""
    _lib.require_device(workspace)
    dev = workspace.device
    P, M, N = workspace.shape
    ws = workspace.contiguous()
    if ws.dtype not in (torch.bfloat16, torch.float32):
        raise RuntimeError("workspace must be bfloat16 or float32")
    result = out if out is not None else torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    b = bias.to(device=dev, dtype=torch.bfloat16).contiguous() if bias is not None else None
    check(lib().ci_splitk_reduce(ptr(ws), int(ws.dtype == torch.bfloat16), P, M, N, ptr(b), ptr(result),
                                 result.stride(0), _lib.stream_handle(dev)))
    return result


def plain_linear_same_order(x, weight_kn, tile_k=1024, tile_n=32, bias=None, workspace=None, segments=1):
    """x[..., K] @ weight_kn[K, N] (+ bias) for an uncompressed bf16 weight, through the fused kernel's
    own contraction: same tiling, same matrix instructions in the same order, same partial sums.  The
    result is bit-identical to `fused_rans_linear` on the compressed form of `weight_kn` (tile
    `tile_k` x 32), which `torch.matmul` is not (other summation order).  A verification aid without
    a counterpart in the reference; slow.  `segments` as given to `fused_rans_linear` (it changes how the
    contraction is split into partial sums).  Above DECODE_ONCE_ABOVE_ROWS rows it does what
    `fused_rans_linear` does there, a library GEMM.  `workspace` as for `fused_rans_linear`: when the contraction is
    split over K, the fp32 partial sums [P, M, N] are left at its start."""
    _lib.require_device(x)
    _lib.require_device(weight_kn)
    if weight_kn.dtype != torch.bfloat16 or weight_kn.dim() != 2:
        raise RuntimeError("weight_kn must be a 2-D bfloat16 tensor [K, N]")
    dev = x.device
    w = weight_kn.contiguous()
    K, N = w.shape
    x2 = _prep_x(x, K)
    M = x2.shape[0]
    if DECODE_ONCE_ABOVE_ROWS is not None and M > DECODE_ONCE_ABOVE_ROWS:
        # what fused_rans_linear computes for this many rows: a library GEMM on the decoded weight
        result = torch.matmul(x2, w)
        if bias is not None:
            result += bias.to(device=dev, dtype=torch.bfloat16)
        return result.view(*x.shape[:-1], N)
    result = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    need = lib().ci_fused_linear_workspace_bytes_segmented(M, K, N, int(tile_k), int(tile_n), 0, int(segments))
    ws, ws_bytes = _pick_workspace(workspace, need, dev)
    b = bias.to(device=dev, dtype=torch.bfloat16).contiguous() if bias is not None else None
    check(lib().ci_plain_linear_same_order(ptr(x2), M, K, N, x2.stride(0), ptr(w), int(tile_k), int(tile_n),
                                           int(segments), ptr(b), ptr(result), result.stride(0), ptr(ws),
                                           C.c_size_t(ws_bytes), _lib.stream_handle(dev)))
    return result.view(*x.shape[:-1], N)


# Names under which the reference exports these ops (comp_inference/__init__.py:39-42).
fused_rans_linear_triton = fused_rans_linear
fused_rans_linear_triton_uncoalesced = fused_rans_linear_uncoalesced
fused_rans_linear_triton_splitk = fused_rans_linear_one_stream  # (defined there, not exported by the reference)


def dense_matmul(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """a[..., K] @ b[K, N] for an uncompressed bf16 weight, bf16 result shaped (*a.shape[:-1], N): the
    reference's dense helper (`triton_matmul`, comp_inference/triton_gemm.py:324-338, a split-K GEMV for
    one row and a block GEMM otherwise, fp32 accumulation).  A plain library GEMM: hipBLASLt through
    torch.matmul, on the GPU only."""
    _lib.require_device(a)
    _lib.require_device(b)
    a2 = a.reshape(-1, a.shape[-1])
    if a2.dtype != torch.bfloat16:
        a2 = a2.to(torch.bfloat16)
    out = torch.matmul(a2, b.to(torch.bfloat16))
    return out.view(*a.shape[:-1], b.shape[1])


triton_matmul = dense_matmul
# its two halves take the rows of `a` already flattened to [M, K] (comp_inference/triton_gemm.py:196-321); one library
# call serves both here
triton_gemv = triton_gemm = dense_matmul
