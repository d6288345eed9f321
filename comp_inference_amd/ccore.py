"""Python face of the native library, shaped like the reference's pybind11 module
`comp_inference.ccore` (src/python_bindings.cpp:59-472): `RansManager`, the result classes,
`decompress` and the pinned-memory helpers, with the same names, argument order and dtypes.
Underneath it is ctypes over the C ABI declared in include/comp_inference_hip.h.
"""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from . import _lib
from ._lib import Tiling, check, lib, ptr


def _dev() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("comp_inference_amd.ccore needs a GPU (gfx950); none is visible")
    return torch.device("cuda", torch.cuda.current_device())


def _np_u16(a) -> np.ndarray:
    if isinstance(a, torch.Tensor):
        a = a.detach().cpu()
        a = a.view(torch.int16).numpy().view(np.uint16) if a.dtype == torch.uint16 else a.numpy()
    return np.ascontiguousarray(a).astype(np.uint16, copy=False)


def _u32_from_cpu(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.uint32).view(np.int32).copy()).view(torch.uint32)


class _Result:
    """Read-only attribute bag (pybind11 `def_readonly`)."""

    def __init__(self, **kw):
        object.__setattr__(self, "_fields", dict(kw))

    def __getattr__(self, name):
        try:
            return self._fields[name]
        except KeyError:
            raise AttributeError(name) from None

    def __setattr__(self, name, value):
        raise AttributeError("can't set attribute")


class TiledTensorCompressResult(_Result):
    """src/python_bindings.cpp:27-42, :150-165"""


class UncoalescedTiledTensorCompressResult(_Result):
    """src/python_bindings.cpp:44-58, :167-190"""


class TensorCompressResult(_Result):
    """src/python_bindings.cpp:15-25, :138-147"""


class CompressResult(_Result):
    """numpy flavour, src/python_bindings.cpp:192-220"""


def _host_tables(freqs: np.ndarray, cdf: np.ndarray):
    tables = np.zeros(256, np.uint32)
    slot_map = np.zeros(4096, np.uint8)
    check(lib().ci_build_tables(freqs.ctypes.data_as(C.c_void_p), cdf.ctypes.data_as(C.c_void_p),
                                tables.ctypes.data_as(C.c_void_p), slot_map.ctypes.data_as(C.c_void_p)))
    return tables, slot_map


def _shape2d(data) -> tuple[int, int]:
    shp = tuple(data.shape)
    return int(shp[0]), int(shp[1]) if len(shp) > 1 else 1  # src/python_bindings.cpp:306-310


class RansManager:
    """src/cpp/rans.hpp:9-90.  Compression runs on the current GPU and, like the reference
    (src/cuda/rans_host.cuh:490, :536), waits for the result; outputs are CPU tensors."""

    def __init__(self, max_data_hint: int = 0):
        self._hint = int(max_data_hint)

    # -- tiled, two streams per column: the default format --------------------------------
    def compress_tiled(self, data, freqs, cdf, tile_height: int, tile_width: int):
        """src/python_bindings.cpp:302-347 -> RansManager::compress_tiled_ilp2."""
        return self._compress_bodies(data, freqs, cdf, tile_height, tile_width, two=True)

    # -- tiled, one stream per column, tile bodies of tile_width bytes a row -----------------
    def compress_tiled_one_stream(self, data, freqs, cdf, tile_height: int, tile_width: int):
        """RansManager::compress_tiled of the C++ class (src/cuda/rans_ops.cu:412-600, kernel
        src/cuda/rans_kernels.cuh:316-391), which the reference's Python module does not bind
        (its `compress_tiled` is the two-stream encoder above).  Same result class; `states` and
        `output_sizes` hold tile_width entries per tile.  Read by `rans_decomp_triton_tiled2` /
        `_tiled_splitk`, `fused_rans_linear_triton_splitk` and `fused_rans_embedding_triton_2`."""
        return self._compress_bodies(data, freqs, cdf, tile_height, tile_width, two=False)

    def _compress_bodies(self, data, freqs, cdf, tile_height: int, tile_width: int, two: bool):
        dev = _dev()
        K, N = _shape2d(data)
        if data.numel() != K * N:
            raise RuntimeError("Input size mismatch in tiled compression")  # rans_host.cuh:462-467
        sym = _lib.as_u8(data, dev).reshape(K, N)
        f, c = _np_u16(freqs), _np_u16(cdf)
        t = Tiling()
        check(lib().ci_tiling_init(C.byref(t), K, N, int(tile_height), int(tile_width), 1 if two else 0))
        s = _lib.stream_handle(dev)
        nb = lib().ci_encode_scratch_bytes(t.num_streams, t.capacity)
        scratch = torch.empty(nb, dtype=torch.uint8, device=dev)
        states = torch.empty(t.num_streams, dtype=torch.int32, device=dev)
        sizes = torch.empty(t.num_streams, dtype=torch.int32, device=dev)
        offs = torch.empty(t.num_tiles, dtype=torch.int32, device=dev)
        lens = torch.empty(t.num_tiles, dtype=torch.int32, device=dev)
        total = C.c_uint64(0)
        encode = lib().ci_encode_tiled_ilp2 if two else lib().ci_encode_tiled_one
        pack = lib().ci_pack_tiled_ilp2 if two else lib().ci_pack_tiled_one
        check(encode(ptr(sym), C.byref(t), f.ctypes.data_as(C.c_void_p), c.ctypes.data_as(C.c_void_p),
                     ptr(scratch), C.c_size_t(nb), ptr(states), ptr(sizes), ptr(offs), ptr(lens),
                     C.byref(total), s))
        stream = torch.empty(total.value, dtype=torch.uint8, device=dev)
        check(pack(ptr(scratch), C.byref(t), ptr(sizes), ptr(offs), ptr(lens), ptr(stream),
                   C.c_uint64(total.value), s))
        tables, slot_map = _host_tables(f, c)
        return TiledTensorCompressResult(
            success=True, stream=stream.cpu(), states=states.cpu().view(torch.uint32),
            tables=_u32_from_cpu(tables), slot_map=torch.from_numpy(slot_map),
            output_sizes=sizes.cpu().view(torch.uint32), num_streams=int(t.num_streams),
            stream_len=int(total.value), tile_offsets=offs.cpu().view(torch.uint32),
            tile_max_lens=lens.cpu().view(torch.uint32), num_tiles_n=int(t.num_tiles_n),
            num_tiles_k=int(t.num_tiles_k), tile_height=int(tile_height), tile_width=int(tile_width))

    # -- tiled, one stream per column, densely packed -----------------------------------------
    def compress_tiled_uncoalesced(self, data, freqs, cdf, tile_height: int, tile_width: int):
        """src/python_bindings.cpp:349-397 -> RansManager::compress_tiled_uncoalesced."""
        dev = _dev()
        K, N = _shape2d(data)
        if data.numel() != K * N:
            raise RuntimeError("Input size mismatch in tiled compression")
        sym = _lib.as_u8(data, dev).reshape(K, N)
        f, c = _np_u16(freqs), _np_u16(cdf)
        t = Tiling()
        check(lib().ci_tiling_init(C.byref(t), K, N, int(tile_height), int(tile_width), 0))
        s = _lib.stream_handle(dev)
        nb = lib().ci_encode_scratch_bytes(t.num_streams, t.capacity)
        scratch = torch.empty(nb, dtype=torch.uint8, device=dev)
        states = torch.empty(t.num_streams, dtype=torch.int32, device=dev)
        sizes = torch.empty(t.num_streams, dtype=torch.int32, device=dev)
        offs = torch.empty(t.num_streams, dtype=torch.int32, device=dev)
        total = C.c_uint64(0)
        check(lib().ci_encode_tiled_dense(ptr(sym), C.byref(t), f.ctypes.data_as(C.c_void_p),
                                          c.ctypes.data_as(C.c_void_p), ptr(scratch), C.c_size_t(nb),
                                          ptr(states), ptr(sizes), ptr(offs), C.byref(total), s))
        stream = torch.empty(total.value, dtype=torch.uint8, device=dev)
        check(lib().ci_pack_tiled_dense(ptr(scratch), C.byref(t), ptr(sizes), ptr(offs), ptr(stream),
                                        C.c_uint64(total.value), s))
        tables, slot_map = _host_tables(f, c)
        return UncoalescedTiledTensorCompressResult(
            success=True, stream=stream.cpu(), states=states.cpu().view(torch.uint32),
            tables=_u32_from_cpu(tables), slot_map=torch.from_numpy(slot_map),
            output_sizes=sizes.cpu().view(torch.uint32), num_streams=int(t.num_streams),
            stream_len=int(total.value), stream_offsets=offs.cpu().view(torch.uint32),
            num_tiles_n=int(t.num_tiles_n), num_tiles_k=int(t.num_tiles_k),
            tile_height=int(tile_height), tile_width=int(tile_width))

    # -- flat (legacy) ---------------------------------------------------------------------------
    def compress(self, data, freqs, cdf, min_block_size: int):
        """src/python_bindings.cpp:225-299 (numpy and tensor overloads)."""
        dev = _dev()
        is_np = isinstance(data, np.ndarray)
        dt = torch.from_numpy(np.ascontiguousarray(data)) if is_np else data
        K, N = _shape2d(dt)
        sym = _lib.as_u8(dt, dev).reshape(K, N)
        f, c = _np_u16(freqs), _np_u16(cdf)
        n_streams, cap = C.c_uint32(0), C.c_uint32(0)
        check(lib().ci_flat_geometry(K, N, int(min_block_size), C.byref(n_streams), C.byref(cap)))
        S = n_streams.value
        s = _lib.stream_handle(dev)
        nb = lib().ci_encode_scratch_bytes(S, cap.value)
        scratch = torch.empty(nb, dtype=torch.uint8, device=dev)
        states = torch.empty(S, dtype=torch.int32, device=dev)
        sizes = torch.empty(S, dtype=torch.int32, device=dev)
        ckpt = torch.empty(S * 128, dtype=torch.int64, device=dev)
        max_len = C.c_uint32(0)
        check(lib().ci_encode_flat(ptr(sym), K, N, S, cap.value, f.ctypes.data_as(C.c_void_p),
                                   c.ctypes.data_as(C.c_void_p), ptr(scratch), C.c_size_t(nb),
                                   ptr(states), ptr(sizes), ptr(ckpt), C.byref(max_len), s))
        stream = torch.empty(max_len.value * S, dtype=torch.uint8, device=dev)
        check(lib().ci_pack_flat(ptr(scratch), S, cap.value, ptr(sizes), max_len.value, ptr(stream), s))
        tables, slot_map = _host_tables(f, c)
        if is_np:
            return CompressResult(
                success=True, stream=stream.cpu().numpy(),
                states=states.cpu().numpy().view(np.uint32),
                output_sizes=sizes.cpu().numpy().view(np.uint32), tables=tables, slot_map=slot_map,
                num_streams=S, stream_len=int(stream.numel()))
        # the tensor overload hands states/sizes back as int32 (src/python_bindings.cpp:261-273)
        return TensorCompressResult(
            success=True, stream=stream.cpu(), states=states.cpu(), output_sizes=sizes.cpu(),
            tables=_u32_from_cpu(tables), slot_map=torch.from_numpy(slot_map),
            checkpoints=ckpt.cpu().view(torch.uint64), num_streams=S, stream_len=int(stream.numel()))

    # -- flat decode through the manager ----------------------------------------------------------
    def decompress(self, stream, states, sizes, num_streams: int, output_len: int, freqs, cdf):
        """src/python_bindings.cpp:399-437 -> (output, kernel milliseconds)."""
        is_np = isinstance(stream, np.ndarray)
        out = (np.empty(output_len, np.uint8) if is_np
               else torch.empty(output_len, dtype=torch.uint8, device=stream.device))
        ms = self.decompress_into(stream, states, sizes, num_streams, freqs, cdf, out)
        return out, ms

    def decompress_into(self, stream, states, sizes, num_streams: int, freqs, cdf, output_buffer):
        """src/python_bindings.cpp:438-471 -> kernel milliseconds.  Host buffers in, host buffer
        out (src/cuda/rans_ops.cu:602-617); the decode itself runs on the GPU."""
        dev = _dev()

        def to_t(a):
            return torch.from_numpy(np.ascontiguousarray(a)) if isinstance(a, np.ndarray) else a

        f, c = _np_u16(freqs), _np_u16(cdf)
        tables, slot_map = _host_tables(f, c)
        d_out = torch.empty(int(np.prod(output_buffer.shape)), dtype=torch.uint8, device=dev)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        d_stream = _lib.as_u8(to_t(stream), dev)
        d_states = _lib.as_u32(to_t(states), dev)
        d_sizes = _lib.as_u32(to_t(sizes), dev)
        d_tables = _u32_from_cpu(tables).to(dev)
        d_slot = torch.from_numpy(slot_map).to(dev)
        start.record()
        decompress(d_stream, d_states, d_sizes, int(num_streams), d_tables, d_slot, d_out)
        stop.record()
        stop.synchronize()
        if isinstance(output_buffer, np.ndarray):
            output_buffer.reshape(-1)[:] = d_out.cpu().numpy()
        else:
            output_buffer.view(-1).copy_(d_out)
        return float(start.elapsed_time(stop))


def decompress(stream, states, sizes, num_streams: int, tables, slot_map, output) -> None:
    """Flat decode, GPU tensors in and out, current stream, no sync
    (src/python_bindings.cpp:61-78 -> src/cuda/rans_ops.cu:619-629): every stream decodes
    ceil(output.numel() / num_streams) symbols; symbol i of stream g lands at output[g + i*num_streams]."""
    if not stream.is_cuda:
        raise RuntimeError("Stream must be on GPU")
    if not output.is_cuda:
        raise RuntimeError("Output buffer must be on GPU")
    _lib.require_device(output)
    dev = output.device
    if states.numel() < int(num_streams) or sizes.numel() < int(num_streams) or tables.numel() != 256 \
            or slot_map.numel() != 4096:
        raise ValueError(f"states and sizes must hold {int(num_streams)} entries, tables 256, slot_map 4096")
    # device copies must stay referenced until the launch has been enqueued
    st, sz = _lib.as_u32(states, dev), _lib.as_u32(sizes, dev)
    tb, sm = _lib.as_u32(tables, dev), _lib.as_u8(slot_map, dev)
    check(lib().ci_decode_flat_strided(
        ptr(stream), C.c_uint64(stream.numel()), ptr(st), ptr(sz), int(num_streams), ptr(tb), ptr(sm),
        C.c_uint64(output.numel()), ptr(output), _lib.stream_handle(dev)))


def allocate_pinned_memory(size: int) -> np.ndarray:
    """Pinned numpy uint8 array (src/python_bindings.cpp:91-104); the tensor that owns the
    pinned allocation stays alive as the array's base."""
    return torch.empty(int(size), dtype=torch.uint8, pin_memory=True).numpy()


def allocate_pinned_tensor(size: int) -> torch.Tensor:
    """Pinned torch uint8 tensor (src/python_bindings.cpp:105-135)."""
    return torch.empty(int(size), dtype=torch.uint8, pin_memory=True)
