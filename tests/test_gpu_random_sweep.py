"""A seeded sweep over shapes, tile heights, weight statistics and segment counts, through the module-level
compressor and every fused operator: decode and gather bit-exact, the two linears bit-identical to the
same contraction on the plain weight and within the reference's allclose(1e-2, 1e-2) of the fp32 product
(for the two weight kinds whose magnitudes span many binades, "wide" and "cols", where sums cancel far
below their terms, the same bar scaled to sum |x||w|).  Weight statistics include the cases that leave the
hand-scheduled paths: near-constant planes (streams of a few bytes), mostly-zero weights, columns of very
different compressibility inside one tile (ragged stream lengths), wide exponent ranges (deep bodies)."""
import random

import pytest
import torch
import torch.nn as nn

pytestmark = pytest.mark.gpu
KINDS = ["normal", "normal", "wide", "const", "sparse", "cols"]


def _weight(K, N, kind, g):
    w = torch.randn(K, N, generator=g)
    if kind == "normal":
        w = w * 0.02
    elif kind == "wide":
        w = w * torch.exp(torch.randn(K, N, generator=g) * 2.0)
    elif kind == "const":
        w = torch.full((K, N), 0.0123)
        w[torch.rand(K, N, generator=g) < 0.001] = 3.5
    elif kind == "sparse":
        w = w * 0.02
        w[torch.rand(K, N, generator=g) < 0.9] = 0.0
    else:
        w = w * 0.02 * torch.exp(torch.randn(1, N, generator=g) * 3.0)
        w[:, torch.rand(N, generator=g) < 0.3] = 0.5
    return w.to(torch.bfloat16).contiguous()


def _compress(ci, w, th, table_layout):
    """-> keyword arguments of the fused entry points, or None when a stream outgrows the encoder's
    capacity (the reference truncates such streams silently, src/cuda/rans_kernels.cuh:140-147)."""
    K, N = w.shape
    if table_layout:
        m = nn.Embedding(K, N).to(torch.bfloat16)
        m.weight.data = w.clone()
    else:
        m = nn.Linear(K, N, bias=False).to(torch.bfloat16)
        m.weight.data = w.t().contiguous()
    try:
        ci.rans_compress_module_weight(m, tile_height=th, tile_width=32, transpose_weight=not table_layout)
    except RuntimeError as e:
        assert "capacity" in str(e)
        return None
    return dict(compressed_data=m.exponent_compressed_weight.cuda(), initial_states=m.exponent_states.cuda(),
                tables=m.exponent_tables.cuda(), slot_map=m.exponent_slot_map.cuda(), weight_shape=(K, N),
                tile_offsets=m.exponent_tile_offsets.cuda(), tile_max_lens=m.exponent_tile_max_lens.cuda(),
                tile_k=th, tile_n=32, mantissas=m.mantissa_raw.cuda())


def _checkpoints(ci, a, segs):
    if segs <= 1:
        return None
    return ci.build_checkpoints(a["compressed_data"], a["initial_states"], a["tables"], a["slot_map"], a["weight_shape"],
                                a["tile_offsets"], a["tile_max_lens"], a["tile_k"], a["tile_n"], segs)


def _same(a, b):
    return torch.equal(a.view(torch.int16), b.view(torch.int16))


def _within(got, x, w_kn, bias, kind):
    want = x.float() @ w_kn.float()
    if bias is not None:
        want = want + bias.float()
    if kind not in ("wide", "cols"):
        return bool(torch.allclose(got.float(), want, atol=1e-2, rtol=1e-2))  # tests/test_mat_mul.py:220,238
    bound = 1e-2 * (x.float().abs() @ w_kn.float().abs()) + 1e-2
    if bias is not None:
        bound = bound + 1e-2 * bias.float().abs()
    return bool(((got.float() - want).abs() <= bound).all())


def _one_case(ci, rng, big):
    g = torch.Generator().manual_seed(rng.randrange(1 << 30))
    op = rng.choice(["linear", "linear", "embed", "trans", "decode"])
    th = rng.choice([64, 128, 256, 512, 1024, 1024, 1024, 2048])
    kind = rng.choice(KINDS)
    segs = rng.choice([s for s in (1, 2, 4, 8) if (th // 2) % (16 * s) == 0])
    if op == "linear":
        K = rng.choice([th, 2 * th, 3 * th, 4 * th, rng.randrange(th, 6 * th), rng.randrange(th, 16 * th)])
        N = rng.choice([32, 64, 96, rng.randrange(32, 700), rng.randrange(32, 3000)])
        M = rng.choice([1, 1, 2, 4, 8, 17, 32, 33, 64, rng.randrange(1, 65), rng.randrange(65, 100)])
        if big:
            th = rng.choice([512, 1024])
            K = th * rng.choice([2, 4, 7, 14]) - rng.choice([0, 0, 5, 300])
            N = rng.choice([4096, rng.randrange(3000, 9000), rng.randrange(9000, 20000)])
            segs = rng.choice([1, 2, 4, 8])
        what = f"linear K={K} N={N} M={M} th={th} {kind} segs={segs}"
        w = _weight(K, N, kind, g)
        a = _compress(ci, w, th, False)
        if a is None:
            return None
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        bias = torch.randn(N, generator=g).to(torch.bfloat16) if rng.random() < 0.3 else None
        bias_d = None if bias is None else bias.cuda()
        got = ci.fused_rans_linear(x.cuda(), **a, bias=bias_d, checkpoints=_checkpoints(ci, a, segs), segments=segs)
        ref = ci.plain_linear_same_order(x.cuda(), w.cuda(), tile_k=th, tile_n=32, bias=bias_d, segments=segs)
        assert _same(got, ref), what
        assert _within(got.cpu(), x, w, bias, kind), what
    elif op == "embed":
        K = rng.choice([th, 2 * th + 5, rng.randrange(th, 5 * th), rng.randrange(th, 40 * th)])
        N = rng.choice([32, 64, 128, rng.randrange(32, 600)])
        T = rng.choice([1, 2, 7, 64, 300, 2048])
        if big:
            th, K, N, T = 1024, rng.randrange(20000, 130000), rng.choice([512, 1024, rng.randrange(500, 3000)]), 2048
            segs = rng.choice([1, 8])
        mode = rng.choice(["uniform", "skewed", "one", "edge"])
        what = f"embed K={K} N={N} T={T} th={th} {kind} segs={segs} ids={mode}"
        w = _weight(K, N, kind, g)
        a = _compress(ci, w, th, True)
        if a is None:
            return None
        if mode == "uniform":
            ids = torch.randint(0, K, (T,), generator=g)
        elif mode == "skewed":
            ids = (torch.rand(T, generator=g) ** 4 * K).long().clamp(max=K - 1)
        elif mode == "one":
            ids = torch.full((T,), rng.randrange(K))
        else:
            edges = [0, K - 1, -1, K, K + 5, th // 2 - 1, th // 2, th - 1, min(th, K - 1)]
            ids = torch.tensor([rng.choice(edges) for _ in range(T)])
        got = ci.fused_rans_embedding(ids.cuda(), **a, checkpoints=_checkpoints(ci, a, segs), segments=segs).cpu()
        ok = (ids >= 0) & (ids < K)
        want = torch.zeros(T, N, dtype=torch.bfloat16)
        want[ok] = w[ids[ok]]
        assert _same(got, want), what
    elif op == "trans":
        V = rng.choice([th, 2 * th, rng.randrange(th, 6 * th), rng.randrange(th, 30 * th)])
        H = rng.choice([32, 64, 256, rng.randrange(32, 500)])
        M = rng.choice([1, 1, 2, 3, 4, 5, 9])
        if big:
            th, V, H = 1024, rng.randrange(20000, 130000), rng.choice([512, 1024, rng.randrange(500, 2048)])
        what = f"transposed V={V} H={H} M={M} th={th} {kind}"
        w = _weight(V, H, kind, g)
        a = _compress(ci, w, th, True)
        if a is None:
            return None
        x = torch.randn(M, H, generator=g).to(torch.bfloat16)
        got = ci.fused_rans_linear_transposed(x.cuda(), **a)
        assert _same(got, ci.plain_linear_transposed_same_order(x.cuda(), w.cuda(), tile_k=th, tile_n=32)), what
        assert _within(got.cpu(), x, w.t(), None, kind), what
    else:
        K = max(th, rng.choice([th, rng.randrange(1, 4 * th), rng.randrange(th, 20 * th)]))
        N = max(32, rng.choice([1, 31, 32, 33, 64, rng.randrange(1, 900)]))
        what = f"decode K={K} N={N} th={th} {kind} segs={segs}"
        w = _weight(K, N, kind, g)
        a = _compress(ci, w, th, True)
        if a is None:
            return None
        exp = ci.rans_decomp_tiled(a["compressed_data"], a["initial_states"], a["tables"], a["slot_map"], (K, N),
                                   a["tile_offsets"], a["tile_max_lens"], th, 32, checkpoints=_checkpoints(ci, a, segs),
                                   segments=segs)
        assert torch.equal(exp.cpu(), ((w.view(torch.int16).to(torch.int32) >> 7) & 0xFF).to(torch.uint8)), what
    return op


@pytest.mark.parametrize("seed,cases,big", [(101, 400, False), (202, 400, False), (303, 12, True)])
def test_random_sweep(always_fused, seed, cases, big):
    import comp_inference_amd as ci

    rng = random.Random(seed)
    done = [_one_case(ci, rng, big) for _ in range(cases)]
    ran = [d for d in done if d is not None]
    assert len(ran) >= cases * 3 // 4 and set(ran) == {"linear", "embed", "trans", "decode"}
