"""The fused decompress-gather on sixteen wavefronts per CU (tables with decoder checkpoints and the slot table
kept beside them): bit exact against table[ids] and against the kernel it stands in for.

Not collected by pytest until it has passed on the GPU (run it by naming the file)."""
import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_weight_kn

pytestmark = pytest.mark.gpu


def _t32(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int32))


class _Table:
    def __init__(self, oracle, K, N, th, segments, seed):
        import comp_inference_amd as ci

        dev = "cuda"
        self.K, self.N, self.th, self.segments = K, N, th, segments
        self.table = make_weight_kn(N, K, seed=seed)  # [K, N], rows are vocabulary entries
        enc, man = oracle.compress_bf16(bf16_bits(self.table), th, 32)
        self.ops = (torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
                    torch.from_numpy(enc.slot_map).to(dev))
        self.meta = (_t32(enc.tile_offsets).to(dev), _t32(enc.tile_max_lens).to(dev))
        self.man = torch.from_numpy(man).to(dev)
        self.ck = ci.build_checkpoints(*self.ops, (K, N), *self.meta, th, 32, segments)
        self.slot_table = ci.build_slot_table(self.ops[2], self.ops[3])

    def gather(self, ids, sixteen: bool):
        import comp_inference_amd as ci

        return ci.fused_rans_embedding(ids.cuda(), *self.ops, (self.K, self.N), *self.meta, self.th, 32, self.man,
                                       checkpoints=self.ck, segments=self.segments,
                                       slot_table=self.slot_table if sixteen else None)

    def expected(self, ids):
        flat = ids.reshape(-1)
        want = torch.zeros(flat.numel(), self.N, dtype=torch.bfloat16)
        ok = (flat >= 0) & (flat < self.K)
        want[ok] = self.table[flat[ok]]
        return want.view(*ids.shape, self.N)


def _check(t, ids):
    got = t.gather(ids, True)
    assert got.shape == (*ids.shape, t.N) and got.dtype == torch.bfloat16
    assert torch.equal(got.cpu().view(torch.int16), t.expected(ids).view(torch.int16))
    assert torch.equal(got, t.gather(ids, False))


@pytest.mark.parametrize("K,N,th,segments", [
    (4096, 256, 1024, 8),    # buckets of 64 rows, whole tiles
    (1300, 128, 1024, 4),    # a short last tile row
    (2048, 96, 1024, 8),     # an odd number of column tiles: the last pair has one tile
    (700, 100, 256, 2),      # ragged columns: the last pair takes the guarded path
    (2048, 64, 512, 2),      # buckets of 128 rows
])
def test_gather_on_sixteen_wavefronts(oracle, K, N, th, segments):
    t = _Table(oracle, K, N, th, segments, seed=K + N)
    rng = np.random.default_rng(4)
    ids = np.concatenate([rng.integers(0, K, 300), [0, K - 1, K, -1, 5, 5, 5, th // 2 - 1, th // 2, min(K - 1, th)]])
    _check(t, torch.from_numpy(ids.astype(np.int64)))
    _check(t, torch.tensor([[K - 1]], dtype=torch.int64))            # one item per pair, nothing to look ahead to
    _check(t, torch.tensor([-3, K, K + 100], dtype=torch.int64))     # only ids outside the table


def test_hot_bucket_and_many_ids(oracle):
    """Thousands of requests for few buckets (chunks of 64 requests, duplicates), more ids than one pass holds."""
    K, N, th = 4096, 128, 1024
    t = _Table(oracle, K, N, th, 8, seed=9)
    rng = np.random.default_rng(1)
    p = 1.0 / np.arange(1, K + 1) ** 1.3
    ids = rng.choice(K, 20000, p=p / p.sum()).astype(np.int64)
    ids[::97] = -1
    _check(t, torch.from_numpy(ids))


def test_every_row_of_a_tile_row(oracle):
    K, N, th = 2048, 64, 1024
    t = _Table(oracle, K, N, th, 8, seed=2)
    _check(t, torch.arange(1024, 2048, dtype=torch.int64))
    _check(t, torch.arange(2047, -1, -1, dtype=torch.int64))


def test_the_module_takes_the_kernel_when_switched_on(oracle):
    import comp_inference_amd as ci

    V, H = 2048, 128
    emb = torch.nn.Embedding(V, H).to(torch.bfloat16)
    with torch.no_grad():
        emb.weight.copy_(make_weight_kn(H, V, seed=6))
    table = emb.weight.detach().clone()
    ci.rans_compress_module_weight(emb, tile_height=1024, tile_width=32, transpose_weight=False)
    mod = ci.RansEmbedding.from_compressed(emb)
    ids = torch.randint(0, V, (3, 50), generator=torch.Generator().manual_seed(1))
    want = table[ids].view(torch.int16)
    assert torch.equal(mod(ids.cuda()).cpu().view(torch.int16), want)
    mod.sixteen_wavefronts = True
    assert torch.equal(mod(ids.cuda()).cpu().view(torch.int16), want)
    assert mod._slot_table_cache[1].numel() == 32768
