"""The first tiled format on the GPU: one stream per column and tile, packed into tile bodies of tile_width
bytes a row (src/cuda/rans_kernels.cuh:316-391 + src/cuda/rans_ops.cu:412-600; consumers in
comp_inference/rans_triton.py:355-516, linear_triton.py:806-1035, embedding_triton.py:8-167).  Encoder bit-exact
against the oracle; decode and gather exact; the two linears within the reference's tolerance of torch.matmul
(tests/test_mat_mul.py:220) and bit-identical to the same kernels on the dense one-stream layout, which holds
the same streams at other addresses.

Not collected by pytest until it has passed on the GPU (run it by naming the file)."""
import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_weight_kn, make_x, zipf_bytes

pytestmark = pytest.mark.gpu

ATOL = RTOL = 1e-2


def _t32(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int32)).view(torch.uint32)


def _np32(t):
    return t.view(torch.int32).numpy().view(np.uint32)


def _u16(a):
    return torch.from_numpy(a.view(np.int16)).view(torch.uint16)


def _operands(enc, dev="cuda"):
    return (torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
            torch.from_numpy(enc.slot_map).to(dev))


@pytest.mark.parametrize("K,N,th,tw", [(1024, 64, 1024, 32), (700, 50, 256, 32), (256, 128, 64, 16), (80, 24, 32, 8),
                                       (2048, 96, 1024, 32)])
def test_one_stream_encode_decode(oracle, K, N, th, tw):
    from comp_inference_amd import ccore, rans_decomp_tiled_one_stream

    sym = zipf_bytes(K * N, 1.5, 3).reshape(K, N)
    f, c = oracle.get_lut(sym)
    ref = oracle.encode_tiled_one(sym, f, c, th, tw)
    got = ccore.RansManager().compress_tiled_one_stream(torch.from_numpy(sym), _u16(f), _u16(c), th, tw)
    assert got.num_streams == ref.num_streams and got.stream_len == ref.stream.size
    assert np.array_equal(got.stream.numpy(), ref.stream)
    assert np.array_equal(_np32(got.states), ref.states)
    assert np.array_equal(_np32(got.output_sizes), ref.sizes)
    assert np.array_equal(_np32(got.tile_offsets), ref.tile_offsets)
    assert np.array_equal(_np32(got.tile_max_lens), ref.tile_max_lens)
    out = rans_decomp_tiled_one_stream(got.stream.cuda(), got.states, got.tables, got.slot_map, (K, N),
                                       got.tile_offsets, got.tile_max_lens, tile_k=th, tile_n=tw)
    assert np.array_equal(out.cpu().numpy(), sym)


def test_one_stream_decode_merges_the_mantissa_plane(oracle):
    from comp_inference_amd import rans_decomp_tiled_one_stream

    K, N, th, tw = 700, 70, 256, 32
    w = make_weight_kn(N, K, seed=41)
    e, m = oracle.split_bf16(bf16_bits(w))
    f, c = oracle.get_lut(e)
    enc = oracle.encode_tiled_one(e, f, c, th, tw)
    man = oracle.interleave_plane(m, th, tw)
    dev = "cuda"
    out = rans_decomp_tiled_one_stream(*_operands(enc), (K, N), _t32(enc.tile_offsets).to(dev),
                                       _t32(enc.tile_max_lens).to(dev), tile_k=th, tile_n=tw,
                                       mantissas=torch.from_numpy(man).to(dev))
    assert torch.equal(out.cpu().view(torch.int16), w.view(torch.int16))


def test_states_of_the_wrong_count_are_refused(oracle):
    """comp_inference/rans_triton.py:482-487"""
    from comp_inference_amd import rans_decomp_tiled_one_stream

    K, N, th, tw = 256, 64, 64, 32
    sym = zipf_bytes(K * N, 1.5, 4).reshape(K, N)
    f, c = oracle.get_lut(sym)
    two = oracle.encode_tiled_ilp2(sym, f, c, th, tw)     # twice the states
    dev = "cuda"
    with pytest.raises(ValueError, match="Initial states size mismatch"):
        rans_decomp_tiled_one_stream(*_operands(two), (K, N), _t32(two.tile_offsets).to(dev),
                                     _t32(two.tile_max_lens).to(dev), tile_k=th, tile_n=tw)


@pytest.mark.parametrize("K,N,th,tw,M", [(1024, 64, 512, 32, 3), (1024, 96, 1024, 32, 1), (700, 64, 1024, 32, 9),
                                         (2048, 256, 1024, 32, 16), (256, 128, 256, 64, 5)])
def test_one_stream_linear(oracle, K, N, th, tw, M):
    from comp_inference_amd import fused_rans_linear_one_stream, fused_rans_linear_triton_uncoalesced

    w = make_weight_kn(N, K, seed=31)
    e, m = oracle.split_bf16(bf16_bits(w))
    f, c = oracle.get_lut(e)
    enc = oracle.encode_tiled_one(e, f, c, th, tw)
    man = torch.from_numpy(oracle.interleave_plane(m, th, tw)).cuda()
    x = make_x(M, K, seed=32).cuda()
    bias = make_x(1, N, seed=33).view(N).cuda()
    dev = "cuda"
    got = fused_rans_linear_one_stream(x, *_operands(enc), (K, N), _t32(enc.tile_offsets).to(dev),
                                       _t32(enc.tile_max_lens).to(dev), th, tw, man, bias=bias)
    want = torch.matmul(x.float().cpu(), w.float()) + bias.float().cpu()
    assert got.shape == (M, N) and got.dtype == torch.bfloat16
    assert torch.allclose(got.float().cpu(), want, atol=ATOL, rtol=RTOL), (got.float().cpu() - want).abs().max()
    dense = oracle.encode_tiled_dense(e, f, c, th, tw)     # the same streams, concatenated
    same = fused_rans_linear_triton_uncoalesced(x, *_operands(dense), (K, N), _t32(dense.stream_offsets).to(dev),
                                                _t32(dense.sizes).to(dev), th, tw, man, bias=bias)
    assert torch.equal(got, same)


def test_one_stream_embedding(oracle):
    from comp_inference_amd import fused_rans_embedding_one_stream

    K, N, th, tw = 600, 70, 256, 32
    table = make_weight_kn(N, K, seed=12)
    e, m = oracle.split_bf16(bf16_bits(table))
    f, c = oracle.get_lut(e)
    enc = oracle.encode_tiled_one(e, f, c, th, tw)
    man = oracle.interleave_plane(m, th, tw)
    ids = torch.tensor([[0, 599, 600, 255], [256, 300, 300, -1]], dtype=torch.int64)
    dev = "cuda"
    got = fused_rans_embedding_one_stream(ids.to(dev), *_operands(enc), (K, N), _t32(enc.tile_offsets).to(dev),
                                          _t32(enc.tile_max_lens).to(dev), th, tw, torch.from_numpy(man).to(dev))
    assert got.shape == (2, 4, N)
    flat = ids.view(-1)
    want = torch.zeros((flat.numel(), N), dtype=torch.bfloat16)
    ok = (flat >= 0) & (flat < K)
    want[ok] = table[flat[ok]]
    assert torch.equal(got.cpu().view(-1, N).view(torch.int16), want.view(torch.int16))


def test_one_stream_transposed_linear(oracle):
    from comp_inference_amd import (fused_rans_linear_transposed_one_stream,
                                    fused_rans_linear_transposed_triton_uncoalesced)

    V, H, th, tw, M = 600, 64, 256, 32, 2
    w = make_weight_kn(H, V, seed=5)
    e, m = oracle.split_bf16(bf16_bits(w))
    f, c = oracle.get_lut(e)
    enc = oracle.encode_tiled_one(e, f, c, th, tw)
    man = torch.from_numpy(oracle.interleave_plane(m, th, tw)).cuda()
    x = make_x(M, H, seed=6).cuda()
    dev = "cuda"
    got = fused_rans_linear_transposed_one_stream(x, *_operands(enc), (V, H), _t32(enc.tile_offsets).to(dev),
                                                  _t32(enc.tile_max_lens).to(dev), th, tw, man)
    want = torch.matmul(x.float().cpu(), w.float().t())
    assert got.shape == (M, V)
    assert torch.allclose(got.float().cpu(), want, atol=ATOL, rtol=RTOL)
    dense = oracle.encode_tiled_dense(e, f, c, th, tw)
    same = fused_rans_linear_transposed_triton_uncoalesced(x, *_operands(dense), (V, H),
                                                           _t32(dense.stream_offsets).to(dev), _t32(dense.sizes).to(dev),
                                                           th, tw, man, workspace=None)
    assert torch.equal(got, same)


def test_one_stream_encoder_and_decoder_on_the_committed_fixture():
    import os

    from comp_inference_amd import ccore, get_rans_lut, rans_decomp_tiled_one_stream

    G = np.load(os.path.join(os.path.dirname(__file__), "golden", "small_formats.npz"))
    K, N, TH, TW = (int(v) for v in G["shape"])
    exp = torch.from_numpy(G["exp"])
    f, c = get_rans_lut(exp)
    t = ccore.RansManager(exp.numel()).compress_tiled_one_stream(exp, f, c, TH, TW)
    assert np.array_equal(t.stream.numpy(), G["one_stream"])
    assert np.array_equal(_np32(t.states), G["one_states"]) and np.array_equal(_np32(t.output_sizes), G["one_sizes"])
    assert np.array_equal(_np32(t.tile_offsets), G["one_tile_offsets"])
    assert np.array_equal(_np32(t.tile_max_lens), G["one_tile_max_lens"])
    dev = "cuda"
    out = rans_decomp_tiled_one_stream(torch.from_numpy(G["one_stream"]).to(dev), _t32(G["one_states"]).to(dev),
                                       _t32(G["tables"]).to(dev), torch.from_numpy(G["slot_map"]).to(dev), (K, N),
                                       _t32(G["one_tile_offsets"]).to(dev), _t32(G["one_tile_max_lens"]).to(dev),
                                       tile_k=TH, tile_n=TW, mantissas=torch.from_numpy(G["man_tiled"]).to(dev))
    assert np.array_equal(out.cpu().view(torch.int16).numpy().view(np.uint16), G["w_bits"])
