"""GPU parity: HIP encoder and decoders against the CPU oracle, bit exact, through the C ABI."""
import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_weight_kn, zipf_bytes

pytestmark = pytest.mark.gpu


def _t32(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int32))


def _np32(t):
    return t.cpu().view(torch.int32).numpy().view(np.uint32)


def _encode_both(oracle, sym, th, tw):
    from comp_inference_amd import ccore, get_rans_lut

    f, c = oracle.get_lut(sym)
    ft, ct = get_rans_lut(torch.from_numpy(sym))
    assert np.array_equal(ft.view(torch.int16).numpy().view(np.uint16), f)
    assert np.array_equal(ct.view(torch.int16).numpy().view(np.uint16), c)
    ref = oracle.encode_tiled_ilp2(sym, f, c, th, tw)
    got = ccore.RansManager(sym.size).compress_tiled(torch.from_numpy(sym), ft, ct, th, tw)
    return ref, got


@pytest.mark.parametrize("K,N,th,tw", [
    (1024, 64, 1024, 32), (2048, 96, 1024, 32), (1300, 80, 1024, 32), (512, 64, 256, 32),
    (96, 100, 32, 32), (256, 128, 64, 16), (384, 256, 128, 64), (256, 256, 256, 128),
])
def test_encoder_matches_oracle(oracle, K, N, th, tw):
    sym = zipf_bytes(K * N, 2.0, K + N).reshape(K, N)
    ref, got = _encode_both(oracle, sym, th, tw)
    assert got.success and got.num_streams == ref.num_streams
    assert np.array_equal(_np32(got.states), ref.states)
    assert np.array_equal(_np32(got.output_sizes), ref.sizes)
    assert np.array_equal(_np32(got.tile_offsets), ref.tile_offsets)
    assert np.array_equal(_np32(got.tile_max_lens), ref.tile_max_lens)
    assert np.array_equal(got.stream.numpy(), ref.stream)
    assert np.array_equal(_np32(got.tables), ref.tables)
    assert np.array_equal(got.slot_map.numpy(), ref.slot_map)
    assert (got.num_tiles_k, got.num_tiles_n) == (ref.num_tiles_k, ref.num_tiles_n)


@pytest.mark.parametrize("K,N,th,tw", [
    (1024, 64, 1024, 32), (4096, 512, 1024, 32), (1300, 80, 1024, 32), (1000, 70, 512, 32),
    (96, 100, 32, 32), (256, 128, 64, 16), (384, 256, 128, 64), (256, 256, 256, 128),
])
def test_tiled_decode_matches_oracle(oracle, K, N, th, tw):
    from comp_inference_amd import rans_decomp_triton_tiled

    w = make_weight_kn(N, K, seed=K * 7 + N)
    e, m = oracle.split_bf16(bf16_bits(w))
    f, c = oracle.get_lut(e)
    enc = oracle.encode_tiled_ilp2(e, f, c, th, tw)
    dev = "cuda"
    args = (torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
            torch.from_numpy(enc.slot_map).to(dev), (K, N), _t32(enc.tile_offsets).to(dev),
            _t32(enc.tile_max_lens).to(dev))
    out = rans_decomp_triton_tiled(*args, tile_k=th, tile_n=tw)
    assert out.dtype == torch.uint8 and tuple(out.shape) == (K, N)
    assert np.array_equal(out.cpu().numpy(), e)
    # merged output: bit-exact bf16 weight
    man = oracle.interleave_plane(m, th, tw)
    wout = rans_decomp_triton_tiled(*args, tile_k=th, tile_n=tw, mantissas=torch.from_numpy(man).to(dev))
    assert np.array_equal(bf16_bits(wout), bf16_bits(w))


def test_batched_decode_matches_oracle(oracle):
    """Several tensors of different shapes (ragged ones included) decoded by one launch."""
    from comp_inference_amd import rans_decomp_tiled_batch

    dev = "cuda"
    shapes = [(2048, 96), (1024, 32), (1300, 80), (4096, 512), (1024, 2048), (512, 40)] * 3  # > 16 items
    items, want = [], []
    for i, (K, N) in enumerate(shapes):
        w = make_weight_kn(N, K, seed=100 + i)
        e, _ = oracle.split_bf16(bf16_bits(w))
        f, c = oracle.get_lut(e)
        enc = oracle.encode_tiled_ilp2(e, f, c, 1024, 32)
        items.append((torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
                      torch.from_numpy(enc.slot_map).to(dev), (K, N), _t32(enc.tile_offsets).to(dev),
                      _t32(enc.tile_max_lens).to(dev)))
        want.append(oracle.decode_tiled_ilp2(enc.stream, enc.states, enc.tables, enc.slot_map, enc.tile_offsets,
                                             enc.tile_max_lens, K, N, 1024, 32))
        assert np.array_equal(want[-1], e)
    outs = rans_decomp_tiled_batch(items, tile_k=1024, tile_n=32)
    assert len(outs) == len(shapes)
    for o, w_, (K, N) in zip(outs, want, shapes):
        assert o.shape == (K, N) and np.array_equal(o.cpu().numpy(), w_)
    assert rans_decomp_tiled_batch([]) == []


@pytest.mark.parametrize("n_sym", [4, 5, 6, 8, 9, 12, 40])
def test_decode_body_depth_classes(oracle, n_sym):
    """Uniform symbols over n_sym values give bodies of about 64 * log2(n_sym) rows: below, between and
    above the depths at which the decoder changes how many tile bodies it keeps in LDS; the last
    values are deeper than any staging area.  One half of the tensor is near-constant so that shallow
    and deep tiles meet in one launch."""
    from comp_inference_amd import rans_decomp_tiled, rans_decomp_tiled_batch

    rng = np.random.default_rng(n_sym)
    K, N = 3072, 96
    e = rng.integers(100, 100 + n_sym, size=(K, N), dtype=np.uint8)
    e[:1024] = np.where(rng.random((1024, N)) < 0.95, 120, e[:1024]).astype(np.uint8)
    f, c = oracle.get_lut(e)
    enc = oracle.encode_tiled_ilp2(e, f, c, 1024, 32)
    dev = "cuda"
    args = (torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
            torch.from_numpy(enc.slot_map).to(dev), (K, N), _t32(enc.tile_offsets).to(dev),
            _t32(enc.tile_max_lens).to(dev))
    assert np.array_equal(rans_decomp_tiled(*args, tile_k=1024, tile_n=32).cpu().numpy(), e)
    a, b = rans_decomp_tiled_batch([args, args], tile_k=1024, tile_n=32)
    assert np.array_equal(a.cpu().numpy(), e) and np.array_equal(b.cpu().numpy(), e)


def test_tiled_decode_state_count_mismatch_raises():
    from comp_inference_amd import rans_decomp_triton_tiled

    z8 = torch.zeros(64, dtype=torch.uint8, device="cuda")
    z32 = torch.zeros(63, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError, match="Initial states size mismatch"):
        rans_decomp_triton_tiled(z8, z32, z32, z8, (1024, 32), z32, z32)


def test_deep_tile_takes_global_path(oracle):
    """Nearly incompressible symbols: tile bodies too deep for the LDS staging area."""
    from comp_inference_amd import rans_decomp_triton_tiled

    K, N = 1024, 64
    sym = np.random.default_rng(5).integers(0, 256, size=(K, N), dtype=np.uint8)
    f, c = oracle.get_lut(sym)
    enc = oracle.encode_tiled_ilp2(sym, f, c, 1024, 32)
    assert enc.tile_max_lens.max() * 64 > 14336
    dev = "cuda"
    out = rans_decomp_triton_tiled(torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev),
                                   _t32(enc.tables).to(dev), torch.from_numpy(enc.slot_map).to(dev), (K, N),
                                   _t32(enc.tile_offsets).to(dev), _t32(enc.tile_max_lens).to(dev))
    assert np.array_equal(out.cpu().numpy(), sym)


@pytest.mark.parametrize("K,N,th,tw", [(1024, 64, 1024, 32), (700, 50, 256, 32), (256, 128, 64, 16)])
def test_dense_encode_decode(oracle, K, N, th, tw):
    from comp_inference_amd import ccore, rans_decomp_tiled_uncoalesced

    sym = zipf_bytes(K * N, 1.5, 3).reshape(K, N)
    f, c = oracle.get_lut(sym)
    ref = oracle.encode_tiled_dense(sym, f, c, th, tw)
    got = ccore.RansManager().compress_tiled_uncoalesced(torch.from_numpy(sym), torch.from_numpy(f.view(np.int16)).view(torch.uint16),
                                                         torch.from_numpy(c.view(np.int16)).view(torch.uint16), th, tw)
    assert np.array_equal(got.stream.numpy(), ref.stream)
    assert np.array_equal(_np32(got.states), ref.states)
    assert np.array_equal(_np32(got.stream_offsets), ref.stream_offsets)
    assert np.array_equal(_np32(got.output_sizes), ref.sizes)
    dev = "cuda"
    out = rans_decomp_tiled_uncoalesced(got.stream.to(dev), got.states, got.tables, got.slot_map, (K, N),
                                        got.stream_offsets, got.output_sizes, tile_k=th, tile_n=tw)
    assert np.array_equal(out.cpu().numpy(), sym)


@pytest.mark.parametrize("K,N", [(300, 8), (512, 33), (1500, 16), (70000, 1)])
def test_flat_encode_decode(oracle, K, N):
    from comp_inference_amd import ccore, rans_decomp_triton

    sym = zipf_bytes(K * N, 4.0, 11).reshape(K, N)
    f, c = oracle.get_lut(sym)
    ref = oracle.encode_flat(sym, f, c, 512)
    got = ccore.RansManager().compress(torch.from_numpy(sym), torch.from_numpy(f.view(np.int16)).view(torch.uint16),
                                       torch.from_numpy(c.view(np.int16)).view(torch.uint16), 512)
    assert got.num_streams == ref.num_streams
    assert got.states.dtype == torch.int32
    assert np.array_equal(got.states.numpy().view(np.uint32), ref.states)
    assert np.array_equal(got.output_sizes.numpy().view(np.uint32), ref.sizes)
    assert np.array_equal(got.stream.numpy(), ref.stream)
    assert np.array_equal(got.checkpoints.view(torch.int64).numpy().view(np.uint64), ref.checkpoints)
    dev = "cuda"
    out = rans_decomp_triton(got.stream.to(dev), got.states.to(dev), got.tables.to(dev), got.slot_map.to(dev),
                             got.output_sizes.to(dev), (K, N))
    assert np.array_equal(out.cpu().numpy(), sym)
    # the extension's own flat decoder writes symbol i of stream g at g + i * streams
    flat = torch.empty(K * N, dtype=torch.uint8, device=dev)
    ccore.decompress(got.stream.to(dev), got.states.to(dev), got.output_sizes.to(dev), got.num_streams,
                     got.tables.to(dev), got.slot_map.to(dev), flat)
    want = oracle.decode_flat_strided(ref.stream, ref.states, ref.sizes, ref.tables, ref.slot_map, K * N)
    assert np.array_equal(flat.cpu().numpy(), want)
    if K <= 512:
        assert np.array_equal(want.reshape(K, N), sym)


def test_tiled_decode_into_caller_tensor(oracle):
    """`out=`: decode in place into a tensor of the caller (exponent plane or merged bf16)."""
    from comp_inference_amd import rans_decomp_tiled

    K, N, th, tw = 1300, 80, 1024, 32
    w = make_weight_kn(N, K, seed=31)
    bits = bf16_bits(w)
    enc, man = oracle.compress_bf16(bits, th, tw)
    dev = "cuda"
    args = (torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
            torch.from_numpy(enc.slot_map).to(dev), (K, N), _t32(enc.tile_offsets).to(dev),
            _t32(enc.tile_max_lens).to(dev))
    e = torch.empty(K, N, dtype=torch.uint8, device=dev)
    assert rans_decomp_tiled(*args, tile_k=th, tile_n=tw, out=e) is e
    assert np.array_equal(e.cpu().numpy(), (bits >> 7).astype(np.uint8))
    b = torch.empty(K, N, dtype=torch.bfloat16, device=dev)
    assert rans_decomp_tiled(*args, tile_k=th, tile_n=tw, mantissas=torch.from_numpy(man).to(dev), out=b) is b
    assert torch.equal(b.cpu().view(torch.int16), w.view(torch.int16))
    with pytest.raises(RuntimeError):
        rans_decomp_tiled(*args, tile_k=th, tile_n=tw, out=b)            # wrong dtype for the exponent plane
    with pytest.raises(RuntimeError):
        rans_decomp_tiled(*args, tile_k=th, tile_n=tw, out=e[:, :40])    # wrong shape


def test_flat_one_column_as_the_reference_script_drives_it(oracle):
    """tests/test_rans.py:55-131 of the reference: numpy bytes of one column through RansManager.compress
    and decompress_into with pinned buffers.  With more than one 512-row segment the extension's strided
    decoder returns the segments transposed (the reference's encoder and decoder disagree,
    src/cuda/rans_kernels.cuh:470-471 against :659-680); the segment-aware decoder returns the data."""
    from comp_inference_amd import ccore, rans_decomp_triton

    size = 4 << 20
    data = zipf_bytes(size, 4.0, 17)
    f, c = oracle.get_lut(data)
    pinned_input, pinned_output = ccore.allocate_pinned_memory(size), ccore.allocate_pinned_memory(size)
    np.copyto(pinned_input, data)
    manager = ccore.RansManager(size)
    res = manager.compress(pinned_input, f, c, 512)
    S = res.num_streams
    assert S == size // 512 and res.stream.size == int(res.output_sizes.max()) * S
    ms = manager.decompress_into(res.stream, res.states, res.output_sizes, S, f, c, pinned_output)
    assert ms > 0
    assert np.array_equal(pinned_output.reshape(512, S), data.reshape(S, 512).T)
    out, _ = manager.decompress(res.stream, res.states, res.output_sizes, S, size, f, c)
    assert np.array_equal(out, pinned_output)
    dev = "cuda"
    tables, slot_map = oracle.build_tables(f, c)
    seg = rans_decomp_triton(torch.from_numpy(res.stream).to(dev), _t32(res.states).to(dev), _t32(tables).to(dev),
                             torch.from_numpy(slot_map).to(dev), _t32(res.output_sizes).to(dev), (size, 1))
    assert np.array_equal(seg.cpu().numpy().reshape(-1), data)


def test_tiled_decode_random_shapes(oracle):
    """Forty seeded random shapes through the 32-column kernels (odd and even numbers of column tiles,
    short last rows and columns, several tile heights): exponent plane and merged bf16 against the oracle."""
    from comp_inference_amd import rans_decomp_tiled

    rng = np.random.default_rng(2024)
    dev = "cuda"
    for case in range(40):
        th = int(rng.choice([64, 256, 1024]))
        K = int(rng.integers(1, 3 * th + 1))
        N = int(rng.integers(1, 200))
        w = make_weight_kn(N, K, seed=1000 + case)
        bits = bf16_bits(w)
        enc, man = oracle.compress_bf16(bits, th, 32)
        args = (torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
                torch.from_numpy(enc.slot_map).to(dev), (K, N), _t32(enc.tile_offsets).to(dev),
                _t32(enc.tile_max_lens).to(dev))
        e = rans_decomp_tiled(*args, tile_k=th, tile_n=32)
        assert np.array_equal(e.cpu().numpy(), (bits >> 7).astype(np.uint8)), (case, K, N, th)
        b = rans_decomp_tiled(*args, tile_k=th, tile_n=32, mantissas=torch.from_numpy(man).to(dev))
        assert torch.equal(b.cpu().view(torch.int16), w.view(torch.int16)), (case, K, N, th)


def test_encoder_random_shapes(oracle):
    """Thirty seeded random planes (shape, tile, skew) through the HIP encoder and packer: every output
    array equals the oracle's, so the stream is the reference's byte for byte."""
    rng = np.random.default_rng(31337)
    overflowed = 0
    for case in range(30):
        th = int(rng.choice([32, 64, 256, 1024]))
        tw = int(rng.choice([16, 32, 32, 64]))
        K = int(rng.integers(1, 3 * th + 1))
        N = int(rng.integers(max(1, tw // 4), 5 * tw))
        sym = zipf_bytes(K * N, float(rng.choice([1.0, 2.0, 4.0])), 5000 + case).reshape(K, N)
        try:
            ref, got = _encode_both(oracle, sym, th, tw)
        except RuntimeError as e:
            # a ragged plane of poorly compressible symbols can outgrow the reference's per-stream
            # capacity (src/cuda/rans_host.cuh:470-471): then both encoders must say so
            assert "capacity" in str(e), (case, K, N, th, tw, str(e))
            from comp_inference_amd import ccore, get_rans_lut

            ft, ct = get_rans_lut(torch.from_numpy(sym))
            with pytest.raises(RuntimeError):
                ccore.RansManager(sym.size).compress_tiled(torch.from_numpy(sym), ft, ct, th, tw)
            overflowed += 1
            continue
        assert got.success and got.num_streams == ref.num_streams, (case, K, N, th, tw)
        assert np.array_equal(_np32(got.states), ref.states), (case, K, N, th, tw)
        assert np.array_equal(_np32(got.output_sizes), ref.sizes), (case, K, N, th, tw)
        assert np.array_equal(_np32(got.tile_offsets), ref.tile_offsets), (case, K, N, th, tw)
        assert np.array_equal(_np32(got.tile_max_lens), ref.tile_max_lens), (case, K, N, th, tw)
        assert np.array_equal(got.stream.numpy(), ref.stream), (case, K, N, th, tw)
    assert overflowed < 10


@pytest.mark.parametrize("K,N,th", [(4096, 256, 1024), (1300, 80, 1024), (2048, 96, 256), (1024, 33, 1024), (700, 64, 64)])
def test_segmented_decode_is_the_same_decode(oracle, K, N, th):
    """Decoder checkpoints only change which wavefront decodes which rows: exponent plane, merged bf16,
    single tensor and batch give the bytes of the unsegmented decode (and of the oracle) for every
    segment count the tile height allows, ragged edges included."""
    from comp_inference_amd import build_checkpoints, rans_decomp_tiled, rans_decomp_tiled_batch

    w = make_weight_kn(N, K, seed=K + N + th)
    e, m = oracle.split_bf16(bf16_bits(w))
    f, c = oracle.get_lut(e)
    enc = oracle.encode_tiled_ilp2(e, f, c, th, 32)
    man = torch.from_numpy(oracle.interleave_plane(m, th, 32)).cuda()
    args = (torch.from_numpy(enc.stream).cuda(), _t32(enc.states).cuda(), _t32(enc.tables).cuda(),
            torch.from_numpy(enc.slot_map).cuda(), (K, N), _t32(enc.tile_offsets).cuda(), _t32(enc.tile_max_lens).cuda())
    plain = rans_decomp_tiled(*args, tile_k=th, tile_n=32)
    assert np.array_equal(plain.cpu().numpy(), e)
    for segs in [s for s in (2, 4, 8) if (th // 2) % (16 * s) == 0]:
        ck = build_checkpoints(*args, tile_k=th, tile_n=32, segments=segs)
        got = rans_decomp_tiled(*args, tile_k=th, tile_n=32, checkpoints=ck, segments=segs)
        assert torch.equal(got, plain), segs
        merged = rans_decomp_tiled(*args, tile_k=th, tile_n=32, mantissas=man, checkpoints=ck, segments=segs)
        assert np.array_equal(bf16_bits(merged), bf16_bits(w)), segs
        a, b = rans_decomp_tiled_batch([args + (ck, segs), args], tile_k=th, tile_n=32)
        assert torch.equal(a, plain) and torch.equal(b, plain), segs
    with pytest.raises(RuntimeError, match="checkpoints"):
        rans_decomp_tiled(*args, tile_k=th, tile_n=32, checkpoints=torch.zeros(3, dtype=torch.int64), segments=2)


def test_segmented_decode_depth_classes(oracle):
    """Shallow, medium and deep bodies (and ones deeper than any staging area) through the segmented
    decode: windows of every class, and items that fall back to guarded reads."""
    from comp_inference_amd import build_checkpoints, rans_decomp_tiled

    for n_sym in (4, 6, 9, 40, 256):
        rng = np.random.default_rng(n_sym)
        K, N = 3072, 96
        e = rng.integers(0 if n_sym == 256 else 100, 256 if n_sym == 256 else 100 + n_sym, size=(K, N), dtype=np.uint8)
        e[:1024] = np.where(rng.random((1024, N)) < 0.95, 120, e[:1024]).astype(np.uint8)
        f, c = oracle.get_lut(e)
        enc = oracle.encode_tiled_ilp2(e, f, c, 1024, 32)
        args = (torch.from_numpy(enc.stream).cuda(), _t32(enc.states).cuda(), _t32(enc.tables).cuda(),
                torch.from_numpy(enc.slot_map).cuda(), (K, N), _t32(enc.tile_offsets).cuda(), _t32(enc.tile_max_lens).cuda())
        for segs in (2, 8):
            ck = build_checkpoints(*args, tile_k=1024, tile_n=32, segments=segs)
            got = rans_decomp_tiled(*args, tile_k=1024, tile_n=32, checkpoints=ck, segments=segs)
            assert np.array_equal(got.cpu().numpy(), e), (n_sym, segs)
