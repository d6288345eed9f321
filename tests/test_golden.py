"""The committed fixture (tests/golden/small_formats.npz, written by tests/golden/make_fixtures.py)
against the oracle, the second Python implementation, the host-side table code and -- on a GPU --
the HIP encoder and decoders."""
import os

import numpy as np
import pytest
import torch

import pyref

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "small_formats.npz"))
K, N, TH, TW = (int(v) for v in G["shape"])


def _t32(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int32))


def test_oracle_reproduces_fixture(oracle):
    exp, man = oracle.split_bf16(G["w_bits"])
    assert np.array_equal(exp, G["exp"]) and np.array_equal(man, G["man"])
    assert np.array_equal(oracle.merge_bf16(exp, man), G["w_bits"])
    freq, cdf = oracle.get_lut(exp)
    assert np.array_equal(freq, G["freq"]) and np.array_equal(cdf, G["cdf"])
    tables, slot_map = oracle.build_tables(freq, cdf)
    assert np.array_equal(tables, G["tables"]) and np.array_equal(slot_map, G["slot_map"])
    t = oracle.encode_tiled_ilp2(exp, freq, cdf, TH, TW)
    assert np.array_equal(t.stream, G["ilp2_stream"]) and np.array_equal(t.states, G["ilp2_states"])
    assert np.array_equal(t.sizes, G["ilp2_sizes"]) and np.array_equal(t.tile_offsets, G["ilp2_tile_offsets"])
    assert np.array_equal(t.tile_max_lens, G["ilp2_tile_max_lens"])
    o = oracle.encode_tiled_one(exp, freq, cdf, TH, TW)
    assert np.array_equal(o.stream, G["one_stream"]) and np.array_equal(o.states, G["one_states"])
    assert np.array_equal(o.sizes, G["one_sizes"]) and np.array_equal(o.tile_offsets, G["one_tile_offsets"])
    assert np.array_equal(o.tile_max_lens, G["one_tile_max_lens"])
    d = oracle.encode_tiled_dense(exp, freq, cdf, TH, TW)
    assert np.array_equal(d.stream, G["dense_stream"]) and np.array_equal(d.states, G["dense_states"])
    assert np.array_equal(d.stream_offsets, G["dense_stream_offsets"])
    f = oracle.encode_flat(exp, freq, cdf, 512)
    assert np.array_equal(f.stream, G["flat_stream"]) and np.array_equal(f.states, G["flat_states"])
    assert np.array_equal(f.sizes, G["flat_sizes"])
    assert np.array_equal(oracle.interleave_plane(man, TH, TW), G["man_tiled"])


def test_decoders_read_fixture(oracle):
    exp = G["exp"]
    assert np.array_equal(oracle.decode_tiled_ilp2(G["ilp2_stream"], G["ilp2_states"], G["tables"], G["slot_map"],
                                                   G["ilp2_tile_offsets"], G["ilp2_tile_max_lens"], K, N, TH, TW), exp)
    assert np.array_equal(pyref.decode_tiled(G["ilp2_stream"], G["ilp2_states"], G["tables"], G["slot_map"],
                                             G["ilp2_tile_offsets"], G["ilp2_tile_max_lens"], K, N, TH, TW), exp)
    one = (G["one_stream"], G["one_states"], G["tables"], G["slot_map"], G["one_tile_offsets"], G["one_tile_max_lens"])
    assert np.array_equal(oracle.decode_tiled_one(*one, K, N, TH, TW), exp)
    assert np.array_equal(pyref.decode_tiled(*one, K, N, TH, TW, halves=1), exp)
    # the same streams as the dense layout holds, at other addresses: states and lengths agree stream for stream
    assert np.array_equal(G["one_states"], G["dense_states"])
    assert np.array_equal(G["one_sizes"],
                          np.diff(np.concatenate([G["dense_stream_offsets"], [G["dense_stream"].size]])))
    sizes = np.diff(np.concatenate([G["dense_stream_offsets"], [G["dense_stream"].size]])).astype(np.uint32)
    assert np.array_equal(oracle.decode_tiled_dense(G["dense_stream"], G["dense_states"], G["tables"], G["slot_map"],
                                                    G["dense_stream_offsets"], sizes, K, N, TH, TW), exp)
    assert np.array_equal(oracle.decode_flat_segmented(G["flat_stream"], G["flat_states"], G["flat_sizes"],
                                                       G["tables"], G["slot_map"], K, N), exp)


def test_host_tables_match_fixture():
    from comp_inference_amd import extract_exp_and_mantissa, get_rans_lut, interleave_mantissas

    w = torch.from_numpy(G["w_bits"].view(np.int16)).view(torch.bfloat16)
    exp, man = extract_exp_and_mantissa(w)
    assert np.array_equal(exp.numpy(), G["exp"]) and np.array_equal(man.numpy(), G["man"])
    f, c = get_rans_lut(exp)
    assert np.array_equal(f.view(torch.int16).numpy().view(np.uint16), G["freq"])
    assert np.array_equal(c.view(torch.int16).numpy().view(np.uint16), G["cdf"])
    assert np.array_equal(interleave_mantissas(man, TH, TW).numpy().reshape(-1), G["man_tiled"].reshape(-1))


@pytest.mark.gpu
def test_hip_encoder_and_decoders_on_fixture():
    from comp_inference_amd import ccore, get_rans_lut, rans_decomp_triton_tiled

    exp = torch.from_numpy(G["exp"])
    f, c = get_rans_lut(exp)
    mgr = ccore.RansManager(exp.numel())
    t = mgr.compress_tiled(exp, f, c, TH, TW)
    assert np.array_equal(t.stream.numpy(), G["ilp2_stream"])
    assert np.array_equal(t.states.view(torch.int32).numpy().view(np.uint32), G["ilp2_states"])
    assert np.array_equal(t.tile_offsets.view(torch.int32).numpy().view(np.uint32), G["ilp2_tile_offsets"])
    assert np.array_equal(t.tile_max_lens.view(torch.int32).numpy().view(np.uint32), G["ilp2_tile_max_lens"])
    d = mgr.compress_tiled_uncoalesced(exp, f, c, TH, TW)
    assert np.array_equal(d.stream.numpy(), G["dense_stream"])
    assert np.array_equal(d.stream_offsets.view(torch.int32).numpy().view(np.uint32), G["dense_stream_offsets"])
    fl = mgr.compress(exp, f, c, 512)
    assert np.array_equal(fl.stream.numpy(), G["flat_stream"])
    dev = "cuda"
    out = rans_decomp_triton_tiled(torch.from_numpy(G["ilp2_stream"]).to(dev), _t32(G["ilp2_states"]).to(dev),
                                   _t32(G["tables"]).to(dev), torch.from_numpy(G["slot_map"]).to(dev), (K, N),
                                   _t32(G["ilp2_tile_offsets"]).to(dev), _t32(G["ilp2_tile_max_lens"]).to(dev),
                                   tile_k=TH, tile_n=TW, mantissas=torch.from_numpy(G["man_tiled"]).to(dev))
    assert np.array_equal(out.cpu().view(torch.int16).numpy().view(np.uint16), G["w_bits"])
