"""Parity at the sizes the benchmarks run at (the seven tensors of one Llama-3-8B-shaped layer, the
128256-row embedding table): bit-exact round trips through the HIP encoder and decoders, the oracle's
stream for a whole tensor, and size-independent properties of the fused operators (tolerance against
torch.matmul, linearity, gather == indexing)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

ATOL = RTOL = 1e-2  # the reference's own bar (tests/test_mat_mul.py:220,238)


LAYER = [("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096),
         ("gate", 14336, 4096), ("up", 14336, 4096), ("down", 4096, 14336)]  # (name, out, in)


@pytest.fixture(scope="module")
def layer_weights():
    """The seven weights of the bench layer, drawn in this order from ONE generator (seed 1), nn.Linear
    orientation, returned transposed to [K=in, N=out]."""
    g = torch.Generator("cpu").manual_seed(1)
    return {name: (torch.randn(o, i, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16).t().contiguous()
            for name, o, i in LAYER}


@pytest.fixture(scope="module")
def gate(layer_weights):
    """gate projection of the bench layer (its fifth draw): [K=4096, N=14336] bf16 N(0, 0.02), compressed on
    the GPU."""
    import comp_inference_amd as ci

    w = layer_weights["gate"]
    exp, man = ci.extract_exp_and_mantissa(w)
    f, c = ci.get_rans_lut(exp)
    r = ci.ccore.RansManager(exp.numel()).compress_tiled(exp, f, c, 1024, 32)
    dev = "cuda"
    d = dict(w=w, exp=exp, f=f, c=c, r=r, man_t=ci.interleave_mantissas(man, 1024, 32).to(dev),
             args=(r.stream.to(dev), r.states.to(dev), r.tables.to(dev), r.slot_map.to(dev), (4096, 14336),
                   r.tile_offsets.to(dev), r.tile_max_lens.to(dev)))
    return d


def test_full_size_encoder_equals_oracle_and_round_trips(oracle, gate):
    import comp_inference_amd as ci

    e = gate["exp"].numpy()
    f, c = oracle.get_lut(e)
    ref = oracle.encode_tiled_ilp2(e, f, c, 1024, 32)
    r = gate["r"]
    assert np.array_equal(r.stream.numpy(), ref.stream)
    assert np.array_equal(r.states.view(torch.int32).numpy().view(np.uint32), ref.states)
    assert np.array_equal(r.tile_max_lens.view(torch.int32).numpy().view(np.uint32), ref.tile_max_lens)
    out = ci.rans_decomp_tiled(*gate["args"], tile_k=1024, tile_n=32)
    assert torch.equal(out.cpu(), gate["exp"])
    both = ci.rans_decomp_tiled_batch([gate["args"], gate["args"]], tile_k=1024, tile_n=32)
    assert torch.equal(both[0], out) and torch.equal(both[1], out)
    w = ci.rans_decomp_tiled(*gate["args"], tile_k=1024, tile_n=32, mantissas=gate["man_t"])
    assert torch.equal(w.cpu().view(torch.int16), gate["w"].view(torch.int16))


def test_whole_layer_decodes_bit_exact_in_one_launch(oracle, layer_weights):
    """Every tensor of the layer: HIP-encoded, decoded by the oracle's decoder and by one batched HIP launch,
    both equal to the exponent plane of the weight; the smallest tensor's stream also byte for byte against
    the oracle's encoder (the largest is compared in the test above)."""
    import comp_inference_amd as ci

    dev = "cuda"
    items, planes = [], []
    for name, w in layer_weights.items():
        exp, _ = ci.extract_exp_and_mantissa(w)
        f, c = ci.get_rans_lut(exp)
        r = ci.ccore.RansManager(exp.numel()).compress_tiled(exp, f, c, 1024, 32)
        u32 = lambda t: t.view(torch.int32).numpy().view(np.uint32)  # noqa: E731
        K, N = w.shape
        back = oracle.decode_tiled_ilp2(r.stream.numpy(), u32(r.states), u32(r.tables), r.slot_map.numpy(),
                                        u32(r.tile_offsets), u32(r.tile_max_lens), K, N, 1024, 32)
        assert np.array_equal(back, exp.numpy()), name
        if name == "k":
            fo, co = oracle.get_lut(exp.numpy())
            ref = oracle.encode_tiled_ilp2(exp.numpy(), fo, co, 1024, 32)
            assert np.array_equal(r.stream.numpy(), ref.stream) and np.array_equal(u32(r.states), ref.states)
        items.append((r.stream.to(dev), r.states.to(dev), r.tables.to(dev), r.slot_map.to(dev), (K, N),
                      r.tile_offsets.to(dev), r.tile_max_lens.to(dev)))
        planes.append(exp)
    outs = ci.rans_decomp_tiled_batch(items, tile_k=1024, tile_n=32)
    for (name, _), o, e in zip(layer_weights.items(), outs, planes):
        assert torch.equal(o.cpu(), e), name
    # the same launch with decoder checkpoints (two segments per stream: sixteen wavefronts per CU on windows of
    # the bodies, what the benchmark times)
    with_ck = [it + (ci.build_checkpoints(*it, 1024, 32, 2), 2) for it in items]
    outs = ci.rans_decomp_tiled_batch(with_ck, tile_k=1024, tile_n=32)
    for (name, _), o, e in zip(layer_weights.items(), outs, planes):
        assert torch.equal(o.cpu(), e), name


@pytest.mark.parametrize("M", [1, 4, 16, 64])
def test_full_size_fused_linear_against_matmul_and_linearity(gate, M):
    import comp_inference_amd as ci

    g = torch.Generator("cpu").manual_seed(2)
    x = torch.randn(64, 4096, generator=g, dtype=torch.float32).to(torch.bfloat16)[:M].contiguous().cuda()
    a = gate["args"]

    def lin(v):
        return ci.fused_rans_linear(v, a[0], a[1], a[2], a[3], (4096, 14336), a[5], a[6], 1024, 32, gate["man_t"])

    y = lin(x).float()
    want = torch.matmul(x.float(), gate["w"].cuda().float())
    assert torch.allclose(y, want, atol=ATOL, rtol=RTOL), float((y - want).abs().max())
    # the operator is linear in x up to bf16 rounding of inputs and outputs
    x2 = torch.randn(M, 4096, generator=g, dtype=torch.float32).to(torch.bfloat16).cuda()
    s = (x.float() + x2.float()).to(torch.bfloat16)
    lhs = lin(s).float()
    rhs = torch.matmul(s.float(), gate["w"].cuda().float())
    assert torch.allclose(lhs, rhs, atol=ATOL, rtol=RTOL)
    # and deterministic: two runs give the same bits
    assert torch.equal(lin(x), lin(x))


def test_full_size_embedding_gather_is_indexing():
    import comp_inference_amd as ci

    V, H = 128256, 4096
    g = torch.Generator("cpu").manual_seed(3)
    table = (torch.randn(V, H, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16)
    exp, man = ci.extract_exp_and_mantissa(table)
    f, c = ci.get_rans_lut(exp)
    r = ci.ccore.RansManager(exp.numel()).compress_tiled(exp, f, c, 1024, 32)
    dev = "cuda"
    p = np.arange(1, V + 1, dtype=np.float64) ** -1.1
    ids = np.random.default_rng(4).choice(V, 2048, p=p / p.sum())
    ids = np.concatenate([ids, [0, V - 1, V - 256, V - 257, 1023, 1024, V, -1]])  # edges of the ragged last tile row
    ids_t = torch.from_numpy(ids.astype(np.int64))
    dargs = (r.stream.to(dev), r.states.to(dev), r.tables.to(dev), r.slot_map.to(dev), (V, H), r.tile_offsets.to(dev),
             r.tile_max_lens.to(dev), 1024, 32)
    man_t = ci.interleave_mantissas(man, 1024, 32).to(dev)
    got = ci.fused_rans_embedding(ids_t.to(dev), *dargs, man_t).cpu()
    ok = (ids_t >= 0) & (ids_t < V)
    want = torch.zeros(ids_t.numel(), H, dtype=torch.bfloat16)
    want[ok] = table[ids_t[ok]]
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # the path RansEmbedding takes by default: decoder checkpoints, 8 segments per stream
    ck = ci.build_checkpoints(*dargs, 8)
    got = ci.fused_rans_embedding(ids_t.to(dev), *dargs, man_t, checkpoints=ck, segments=8).cpu()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # the same table as LM head: logits of one hidden state against torch on the bf16 table
    h = torch.randn(1, H, generator=g, dtype=torch.float32).to(torch.bfloat16)
    logits = ci.fused_rans_linear_transposed(h.to(dev), r.stream.to(dev), r.states.to(dev), r.tables.to(dev),
                                             r.slot_map.to(dev), (V, H), r.tile_offsets.to(dev), r.tile_max_lens.to(dev),
                                             1024, 32, ci.interleave_mantissas(man, 1024, 32).to(dev), None).float().cpu()
    ref = h.float() @ table.float().t()
    assert torch.allclose(logits, ref, atol=ATOL, rtol=RTOL), float((logits - ref).abs().max())
