"""GPU parity of the fused decompress-gather: bit exact against table[ids] and against the oracle's
literal restatement of the reference kernel."""
import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_weight_kn

pytestmark = pytest.mark.gpu


def _t32(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int32))


def _gather(enc, man, ids, K, N, th, tw, **kw):
    from comp_inference_amd import fused_rans_embedding_triton

    dev = "cuda"
    return fused_rans_embedding_triton(
        ids.to(dev), torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
        torch.from_numpy(enc.slot_map).to(dev), (K, N), _t32(enc.tile_offsets).to(dev),
        _t32(enc.tile_max_lens).to(dev), th, tw, torch.from_numpy(man).to(dev), **kw)


def _expected(table, ids):
    K, N = table.shape
    flat = ids.reshape(-1)
    want = torch.zeros(flat.numel(), N, dtype=torch.bfloat16)
    ok = (flat >= 0) & (flat < K)
    want[ok] = table[flat[ok]]
    return want.view(*ids.shape, N)


@pytest.mark.parametrize("K,N,th,tw", [(1300, 128, 1024, 32), (2048, 96, 1024, 32), (700, 64, 256, 32),
                                       (300, 40, 64, 16), (512, 128, 128, 64)])
def test_embedding_matches_table_and_oracle(oracle, K, N, th, tw):
    table = make_weight_kn(N, K, seed=K)  # [K, N], rows are vocabulary entries
    enc, man = oracle.compress_bf16(bf16_bits(table), th, tw)
    rng = np.random.default_rng(4)
    ids = np.concatenate([rng.integers(0, K, 200), [0, K - 1, K, -1, 5, 5, 5, th // 2 - 1, th // 2, min(K - 1, th)]])
    ids_t = torch.from_numpy(ids.astype(np.int64))
    got = _gather(enc, man, ids_t, K, N, th, tw)
    assert got.shape == (ids.size, N) and got.dtype == torch.bfloat16
    want = _expected(table, ids_t)
    assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16))
    ref = oracle.embedding_gather(ids, enc, man, K, N)
    assert np.array_equal(bf16_bits(got), ref)


def test_embedding_single_id_2d_shape_and_out(oracle):
    K, N, th, tw = 1300, 128, 1024, 32
    table = make_weight_kn(N, K, seed=3)
    enc, man = oracle.compress_bf16(bf16_bits(table), th, tw)
    one = torch.tensor([777], dtype=torch.int64)
    assert torch.equal(_gather(enc, man, one, K, N, th, tw).cpu().view(torch.int16),
                       table[777:778].view(torch.int16))
    ids = torch.tensor([[1, 2, 1299], [1024, 0, 511]], dtype=torch.int64)
    out = torch.full((6, N), 7.0, dtype=torch.bfloat16, device="cuda")
    got = _gather(enc, man, ids, K, N, th, tw, out=out)
    assert got.shape == (2, 3, N)
    assert torch.equal(out.cpu().view(torch.int16), _expected(table, ids).view(6, N).view(torch.int16))
    # int32 ids are accepted
    got32 = _gather(enc, man, ids.to(torch.int32), K, N, th, tw)
    assert torch.equal(got32.cpu().view(torch.int16), _expected(table, ids).view(torch.int16))


def test_embedding_more_ids_than_one_sort_pass(oracle):
    K, N, th, tw = 640, 64, 128, 32
    table = make_weight_kn(N, K, seed=8)
    enc, man = oracle.compress_bf16(bf16_bits(table), th, tw)
    rng = np.random.default_rng(0)
    p = 1.0 / np.arange(1, K + 1) ** 1.1
    ids = torch.from_numpy(rng.choice(K, 20000, p=p / p.sum()).astype(np.int64))
    got = _gather(enc, man, ids, K, N, th, tw)
    assert torch.equal(got.cpu().view(torch.int16), table[ids].view(torch.int16))


def test_embedding_hot_bucket_is_split_between_wavefronts(oracle):
    """Thousands of requests for one half tile of rows (with duplicates, invalid ids between them):
    the requests are served in runs of 64 by different wavefronts, each decoding from the top."""
    K, N, th, tw = 2048, 128, 1024, 32
    table = make_weight_kn(N, K, seed=21)
    enc, man = oracle.compress_bf16(bf16_bits(table), th, tw)
    rng = np.random.default_rng(21)
    ids = np.concatenate([rng.integers(0, 400, 3000), rng.integers(500, 530, 300), [-5, K + 7, 2047, 1024, 1535, 1536]])
    rng.shuffle(ids)
    ids_t = torch.from_numpy(ids.astype(np.int64))
    got = _gather(enc, man, ids_t, K, N, th, tw)
    assert torch.equal(got.cpu().view(torch.int16), _expected(table, ids_t).view(torch.int16))


def test_embedding_dense_layout(oracle):
    from comp_inference_amd import fused_rans_embedding_triton_uncoalesced

    K, N, th, tw = 600, 64, 256, 32
    table = make_weight_kn(N, K, seed=12)
    e, m = oracle.split_bf16(bf16_bits(table))
    f, c = oracle.get_lut(e)
    enc = oracle.encode_tiled_dense(e, f, c, th, tw)
    man = oracle.interleave_plane(m, th, tw)
    ids = torch.tensor([0, 599, 600, 255, 256, 300, 300], dtype=torch.int64)
    dev = "cuda"
    got = fused_rans_embedding_triton_uncoalesced(
        ids.to(dev), torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
        torch.from_numpy(enc.slot_map).to(dev), (K, N), _t32(enc.stream_offsets).to(dev), _t32(enc.sizes).to(dev),
        th, tw, torch.from_numpy(man).to(dev))
    assert torch.equal(got.cpu().view(torch.int16), _expected(table, ids).view(torch.int16))


def test_embedding_random_shapes(oracle):
    """Twenty seeded random tables and id lists (duplicates, invalid ids, ragged shapes, three tile heights)."""
    from comp_inference_amd import fused_rans_embedding_triton

    rng = np.random.default_rng(99)
    dev = "cuda"
    for case in range(20):
        th = int(rng.choice([64, 256, 1024]))
        K = int(rng.integers(1, 3 * th + 1))
        N = int(rng.integers(8, 200))   # (fewer real columns than 8 of 32 overrun the reference's stream capacity)
        T = int(rng.integers(1, 300))
        table = make_weight_kn(K, N, seed=4000 + case).t().contiguous()  # [K rows, N columns]
        assert tuple(table.shape) == (K, N)
        enc, man = oracle.compress_bf16(bf16_bits(table), th, 32)
        ids = rng.integers(-2, K + 2, T)
        got = fused_rans_embedding_triton(
            torch.from_numpy(ids).to(dev), torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev),
            _t32(enc.tables).to(dev), torch.from_numpy(enc.slot_map).to(dev), (K, N), _t32(enc.tile_offsets).to(dev),
            _t32(enc.tile_max_lens).to(dev), th, 32, torch.from_numpy(man).to(dev))
        want = torch.zeros(T, N, dtype=torch.bfloat16)
        ok = (ids >= 0) & (ids < K)
        want[torch.from_numpy(ok)] = table[torch.from_numpy(ids[ok])]
        assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16)), (case, K, N, T, th)


@pytest.mark.parametrize("K,N,th,segments", [(1300, 128, 1024, 8), (2048, 96, 1024, 4), (2048, 96, 1024, 16),
                                             (700, 64, 256, 2), (3000, 160, 1024, 8)])
def test_embedding_with_checkpoints(oracle, K, N, th, segments):
    """With decoder checkpoints the gather starts every walk at a segment boundary: same rows, bit for bit
    (ragged shapes, duplicates, invalid ids, hot segments with more than 64 requests)."""
    from comp_inference_amd import build_checkpoints

    table = make_weight_kn(K, N, seed=K + segments).t().contiguous()
    enc, man = oracle.compress_bf16(bf16_bits(table), th, 32)
    rng = np.random.default_rng(K + N)
    ids = np.concatenate([rng.integers(0, K, 400), np.full(150, min(K - 1, 70)), [0, K - 1, K, -1, th // 2 - 1,
                          th // 2, min(K - 1, th), min(K - 1, th // 2 // segments)], rng.integers(60, 70, 100)])
    ids = torch.from_numpy(ids)
    dev = "cuda"
    ck = build_checkpoints(torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
                           torch.from_numpy(enc.slot_map).to(dev), (K, N), _t32(enc.tile_offsets).to(dev),
                           _t32(enc.tile_max_lens).to(dev), th, 32, segments)
    got = _gather(enc, man, ids, K, N, th, 32, checkpoints=ck, segments=segments)
    assert torch.equal(got.cpu().view(torch.int16), _expected(table, ids).view(torch.int16))
    plain = _gather(enc, man, ids, K, N, th, 32)
    assert torch.equal(got, plain)


@pytest.mark.parametrize("K,th", [(530000, 1024), (530000, 64), (300000, 32)])
def test_tables_with_many_rows_and_buckets(K, th):
    """How the requests of a pass are put in order depends on the table: by counting per bucket while the
    counters fit the LDS (530,000 rows under 1024-row tiles), else by a full sort whose elements are one
    word (row << 13 | position) while rows fit 19 bits (300,000 rows, 16-row buckets) and (row, position)
    pairs beyond (530,000 rows, 32-row buckets).  All give table[ids]: duplicates, the last row, invalid
    ids, more ids than one pass holds."""
    import torch.nn as nn

    import comp_inference_amd as ci

    N = 32
    g = torch.Generator().manual_seed(8)
    table = (torch.randn(K, N, generator=g) * 0.02).to(torch.bfloat16)
    emb = nn.Embedding(K, N).to(torch.bfloat16)
    emb.weight.data = table.clone()
    ci.rans_compress_module_weight(emb, tile_height=th, tile_width=32, transpose_weight=False)
    mod = ci.RansEmbedding.from_compressed(emb).cuda()
    assert mod.tile_k == th
    ids = torch.cat([torch.randint(0, K, (9000,), generator=g), torch.tensor([K - 1, 0, K, -3, 262143, 262144, 7, 7]),
                     torch.randint(0, 40, (300,), generator=g)])
    for segments in (1, "auto"):
        mod.segments = segments
        got = mod(ids.cuda()).cpu()
        assert torch.equal(got.view(torch.int16), _expected(table, ids).view(torch.int16)), segments
