"""Host-side weight compression API, mirroring comp_inference/comp_inference.py of the reference:
bf16 plane split/merge, the 12-bit frequency table, the sign|mantissa tile interleave, and the
module-level compress / decompress helpers.  The coding itself runs on the GPU through
`ccore.RansManager` and the HIP decode ops.
"""
from __future__ import annotations

from typing import Tuple

import numpy as np
import torch
import torch.nn as nn

from . import ccore
from .rans_hip import rans_decomp_tiled, rans_decomp_tiled_uncoalesced


def extract_exp_and_mantissa(tensor: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """bf16 -> (exponent plane u8, sign|mantissa plane u8)   [comp_inference.py:10-32]
    exponent = bits 14..7; sign|mantissa = bit 15 moved to bit 7, bits 6..0 kept."""
    if tensor.dtype != torch.bfloat16:
        raise ValueError("Only bfloat16 dtype is supported for exponent/mantissa extraction.")
    raw = tensor.contiguous().view(torch.int16).to(torch.int32) & 0xFFFF
    exponent = (raw >> 7) & 0xFF
    mantissa = ((raw >> 15) << 7) | (raw & 0x7F)
    return exponent.to(torch.uint8), mantissa.to(torch.uint8)


def reconstruct_from_exp_and_mantissa(exponent, mantissa_and_sign, dtype=torch.bfloat16):
    """(exponent u8, sign|mantissa u8) -> bf16   [comp_inference.py:156-180]"""
    e = exponent.to(torch.int32)
    m = mantissa_and_sign.to(torch.int32)
    bits = ((m & 0x80) << 8) | (e << 7) | (m & 0x7F)
    # bits is in [0, 65535]; go through int16 two's complement to reach the 16-bit pattern
    bits = torch.where(bits >= 32768, bits - 65536, bits).to(torch.int16)
    return bits.view(dtype)


def interleave_mantissas(mantissas: torch.Tensor, TILE_K=1024, TILE_N=32):
    """[K,N] -> flat tile-major plane: zero-pad to tile multiples, element (r,c) of tile
    (tk,tn) at (tk*tiles_n + tn)*TILE_K*TILE_N + r*TILE_N + c   [comp_inference.py:35-64]"""
    assert mantissas.is_contiguous(), "Mantissas tensor must be contiguous for interleaving."
    K, N = mantissas.shape
    tiles_k = (K + TILE_K - 1) // TILE_K
    tiles_n = (N + TILE_N - 1) // TILE_N
    pad_k, pad_n = tiles_k * TILE_K - K, tiles_n * TILE_N - N
    if pad_k or pad_n:
        mantissas = torch.nn.functional.pad(mantissas, (0, pad_n, 0, pad_k))
    tiled = mantissas.view(tiles_k, TILE_K, tiles_n, TILE_N).permute(0, 2, 1, 3).contiguous()
    return tiled.view(-1)


def uninterleave_mantissas(interleaved_mantissas, K, N, TILE_K=1024, TILE_N=32):
    """Inverse of interleave_mantissas; a truncated tail is read as zero padding
    [comp_inference.py:67-93]"""
    tiles_k = (K + TILE_K - 1) // TILE_K
    tiles_n = (N + TILE_N - 1) // TILE_N
    expected = tiles_k * tiles_n * TILE_K * TILE_N
    flat = interleaved_mantissas.reshape(-1)
    if flat.numel() < expected:
        flat = torch.nn.functional.pad(flat, (0, expected - flat.numel()))
    tiled = flat[:expected].view(tiles_k, tiles_n, TILE_K, TILE_N).permute(0, 2, 1, 3).contiguous()
    return tiled.view(tiles_k * TILE_K, tiles_n * TILE_N)[:K, :N]


def interleave_mantissas_ilp2(mantissas: torch.Tensor, TILE_K=128, TILE_N=64):
    """[K,N] -> flat tile-major plane with each tile stored as its top half (rows 0 .. TILE_K/2) followed by its
    bottom half   [comp_inference.py:96-129].  Element-for-element the same bytes as `interleave_mantissas` (a tile's
    halves already follow each other there); the reference keeps the name but calls it nowhere (its two call sites
    are comments, comp_inference.py:453, :463).  Defaults as the reference's: 128 x 64."""
    assert TILE_K % 2 == 0, "a tile has two halves"
    return interleave_mantissas(mantissas.contiguous(), TILE_K=TILE_K, TILE_N=TILE_N)


def uninterleave_mantissas_ilp2(interleaved, K, N, TILE_K=128, TILE_N=64):
    """Inverse of interleave_mantissas_ilp2   [comp_inference.py:132-153]."""
    assert TILE_K % 2 == 0, "a tile has two halves"
    return uninterleave_mantissas(interleaved, K, N, TILE_K=TILE_K, TILE_N=TILE_N)


def get_rans_lut(data: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """12-bit frequency and exclusive-cdf tables of a u8 tensor   [comp_inference.py:183-239]
    floor(count/total*4096) in float64, zero -> 1, then the surplus goes to the first maximum or
    the deficit is taken one unit at a time from the current first maximum."""
    flat = data.detach().cpu().contiguous().view(-1)
    if flat.dtype != torch.uint8:
        flat = flat.to(torch.uint8)
    counts = np.bincount(flat.numpy(), minlength=256)
    target = 4096
    freqs = np.floor(counts / counts.sum() * target).astype(np.int32)
    freqs[freqs == 0] = 1
    diff = target - int(freqs.sum())
    if diff > 0:
        freqs[np.argmax(freqs)] += diff
    else:
        while diff < 0:
            idx = int(np.argmax(freqs))
            freqs[idx] -= 1
            assert freqs[idx] >= 1, "Frequency for a symbol dropped to zero, which should not happen."
            diff += 1
    assert int(freqs.sum()) == target
    cdf = np.concatenate(([0], np.cumsum(freqs)[:-1])).astype(np.int32)
    return (torch.from_numpy(freqs.astype(np.uint16).view(np.int16)).view(torch.uint16),
            torch.from_numpy(cdf.astype(np.uint16).view(np.int16)).view(torch.uint16))


def _fuse_and_compress(weights, tile_height, tile_width, uncoalesced_interleaving):
    fused = torch.cat(list(weights), dim=0).contiguous()
    proj = nn.Linear(fused.shape[1], fused.shape[0], bias=False, device=fused.device, dtype=fused.dtype)
    proj.weight = nn.Parameter(fused, requires_grad=False)
    rans_compress_module_weight_bf16(proj, tile_height=tile_height, tile_width=tile_width,
                                     uncoalesced_interleaving=uncoalesced_interleaving)
    return proj


def rans_compress_qkv_fused(self_attn_module: nn.Module, tile_height=1024, tile_width=32,
                            uncoalesced_interleaving=False):
    """Concatenate q/k/v along the output dimension, compress as one weight, keep it under the
    name q_proj and drop k_proj / v_proj   [comp_inference.py:242-293]"""
    q, k, v = (self_attn_module.q_proj.weight, self_attn_module.k_proj.weight,
               self_attn_module.v_proj.weight)
    assert q.dtype == k.dtype == v.dtype == torch.bfloat16
    assert q.shape[1] == k.shape[1] == v.shape[1]
    self_attn_module.q_proj = _fuse_and_compress((q, k, v), tile_height, tile_width,
                                                 uncoalesced_interleaving)
    self_attn_module.qkv_fused = True
    del self_attn_module.k_proj
    del self_attn_module.v_proj


def rans_compress_gate_up_fused(ffn_module: nn.Module, tile_height=1024, tile_width=32,
                                uncoalesced_interleaving=False):
    """Concatenate gate/up, compress as one weight under the name gate_proj, drop up_proj
    [comp_inference.py:296-341]"""
    gate, up = ffn_module.gate_proj.weight, ffn_module.up_proj.weight
    assert gate.dtype == up.dtype == torch.bfloat16
    ffn_module.gate_proj = _fuse_and_compress((gate, up), tile_height, tile_width,
                                              uncoalesced_interleaving)
    ffn_module.gate_up_fused = True
    del ffn_module.up_proj


def rans_compress_module_weight_bf16(module: nn.Module, skip_mantissa=True, tile_height=1024,
                                     tile_width=32, transpose_weight=True,
                                     uncoalesced_interleaving=False) -> None:
    """Compress `module.weight` in place of the weight   [comp_inference.py:344-502]

    The exponent plane is rANS-coded per tile; the sign|mantissa plane is kept raw, tile
    interleaved.  Attribute names are those the reference attaches (`exponent_*`,
    `mantissa_raw`, `input_shape`, `expanded_size`, `compressed`), which its savers and tests read.
    `skip_mantissa=False` (coding the mantissa plane too) is not offered: that branch of the
    reference cannot run (it reads an undefined name, comp_inference.py:435)."""
    if not hasattr(module, "weight"):
        return
    if module.weight.dtype != torch.bfloat16:
        print(f"Skipping {module.weight.dtype}, expected bfloat16.")
        return
    if not skip_mantissa:
        raise NotImplementedError("only the raw sign|mantissa plane (skip_mantissa=True) is supported")
    weight = module.weight.detach()
    if transpose_weight:
        weight = weight.t()
    weight = weight.contiguous()  # [K, N]
    K, N = weight.shape
    if tile_height > K or tile_width > N:
        # The reference shrinks the tile after encoding with the nominal one and returns
        # streams that its own decoders cannot read (src/cuda/rans_ops.cu:219-223).
        raise ValueError(f"tile {tile_height}x{tile_width} is larger than the weight {K}x{N}")
    module.input_shape = [K, N]
    module.expanded_size = weight.numel()

    exponent, mantissa = extract_exp_and_mantissa(weight)
    module.exponent_freqs, module.exponent_cdf = get_rans_lut(exponent)
    module.mantissa_freqs, module.mantissa_cdf = get_rans_lut(mantissa)

    manager = ccore.RansManager(module.expanded_size)
    if uncoalesced_interleaving:
        res = manager.compress_tiled_uncoalesced(exponent, module.exponent_freqs, module.exponent_cdf,
                                                 tile_height, tile_width)
    else:
        res = manager.compress_tiled(exponent, module.exponent_freqs, module.exponent_cdf,
                                     tile_height, tile_width)
    module.exponent_compressed_weight = res.stream
    module.exponent_states = res.states
    module.exponent_output_sizes = res.output_sizes
    module.exponent_num_streams = res.num_streams
    module.exponent_tables = res.tables
    module.exponent_slot_map = res.slot_map
    module.exponent_num_tiles_n = res.num_tiles_n
    module.exponent_num_tiles_k = res.num_tiles_k
    module.exponent_tile_height = res.tile_height
    module.exponent_tile_width = res.tile_width
    module.exponent_uncoalesced_interleaving = bool(uncoalesced_interleaving)
    if uncoalesced_interleaving:
        module.exponent_stream_offsets = res.stream_offsets
    else:
        module.exponent_tile_offsets = res.tile_offsets
        module.exponent_tile_max_lens = res.tile_max_lens

    module.mantissa_raw = interleave_mantissas(mantissa.cpu().contiguous(), TILE_K=tile_height,
                                               TILE_N=tile_width).contiguous()
    module.compressed = "rans_bfloat16"
    del module.weight


def rans_compress_module_weight(module: nn.Module, tile_height=1024, tile_width=32,
                                transpose_weight=True, uncoalesced_interleaving=False) -> None:
    """Dispatcher   [comp_inference.py:548-570]; only bf16 weights are compressed.  The reference also names a
    branch for uint8 / int8 weights (`rans_compress_module_weight_int8`, comp_inference.py:505-545, and its
    decompressor :716-752); neither can run there (the flat `compress` is called without its required
    `min_block_size`, src/python_bindings.cpp:225-228, and the decompressor asks for the `weight` the compressor
    deleted), so there is no behaviour to reproduce and such weights are skipped with the same message."""
    if not hasattr(module, "weight"):
        return
    if module.weight.dtype == torch.bfloat16:
        rans_compress_module_weight_bf16(module, tile_height=tile_height, tile_width=tile_width,
                                         transpose_weight=transpose_weight,
                                         uncoalesced_interleaving=uncoalesced_interleaving)
    else:
        print(f"Module weight dtype is {module.weight.dtype}, not supported for RANS compression. Skipping.")


def compressed_nbytes(module: nn.Module) -> int:
    """Stored bytes of a compressed module: stream + raw plane + per-stream and per-tile metadata."""
    n = module.exponent_compressed_weight.numel() + module.mantissa_raw.numel()
    n += 4 * module.exponent_states.numel() + 1024 + 4096
    if module.exponent_uncoalesced_interleaving:
        n += 4 * module.exponent_stream_offsets.numel()
    else:
        n += 4 * (module.exponent_tile_offsets.numel() + module.exponent_tile_max_lens.numel())
    return int(n)


def rans_decompress_module_weight_bf16(module: nn.Module, device=None) -> None:
    """Rebuild `module.weight` ([K,N], bf16) from the compressed attributes
    [comp_inference.py:573-716].  Tile sizes come from the module (the reference hard-codes
    1024x32 here, comp_inference.py:643-644, :694-696)."""
    if not hasattr(module, "compressed"):
        print("Module is not compressed. Skipping decompression.")
        return
    if module.compressed != "rans_bfloat16":
        print(f"Skipping {module.compressed}, expected rans_bfloat16.")
        return
    shape = module.input_shape
    dev = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
    th = getattr(module, "exponent_tile_height", 1024)
    tw = getattr(module, "exponent_tile_width", 32)
    if getattr(module, "exponent_uncoalesced_interleaving", False):
        offs = module.exponent_stream_offsets.to(torch.int64)
        total = module.exponent_compressed_weight.numel()
        sizes = torch.diff(offs, append=torch.tensor([total], dtype=torch.int64)).to(torch.int32)
        weight = rans_decomp_tiled_uncoalesced(
            module.exponent_compressed_weight.to(dev), module.exponent_states, module.exponent_tables,
            module.exponent_slot_map, shape, module.exponent_stream_offsets, sizes, tile_k=th, tile_n=tw,
            mantissas=module.mantissa_raw)
    else:
        weight = rans_decomp_tiled(
            module.exponent_compressed_weight.to(dev), module.exponent_states, module.exponent_tables,
            module.exponent_slot_map, shape, module.exponent_tile_offsets, module.exponent_tile_max_lens,
            tile_k=th, tile_n=tw, mantissas=module.mantissa_raw)
    module.weight = weight


def rans_decompress_module_weight(module: nn.Module, device=None) -> None:
    """Dispatcher   [comp_inference.py:754-778]: restores `module.weight` as an nn.Parameter."""
    if not hasattr(module, "compressed"):
        return
    if module.compressed == "rans_bfloat16":
        rans_decompress_module_weight_bf16(module, device=device)
    else:
        print(f"Unknown compression type: {module.compressed}")
        return
    if not isinstance(module.weight, nn.Parameter):
        module.weight = nn.Parameter(module.weight, requires_grad=False)
