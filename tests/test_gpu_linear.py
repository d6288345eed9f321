"""GPU parity of the fused decompress-linear: against torch.matmul on the oracle-decoded weight,
with the tolerance the reference's own test uses (tests/test_mat_mul.py:220: atol=rtol=1e-2)."""
import numpy as np
import pytest
import torch

from helpers import bf16_bits, bits_to_bf16, make_weight_kn, make_x

pytestmark = pytest.mark.gpu
ATOL = RTOL = 1e-2


def _t32(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int32))


def _compress(oracle, w, th, tw):
    enc, man = oracle.compress_bf16(bf16_bits(w), th, tw)
    K, N = w.shape
    wdec = bits_to_bf16(oracle.decompress_bf16(enc, man, K, N))
    assert torch.equal(wdec.view(torch.int16), w.view(torch.int16))
    return enc, man, wdec


def _call(enc, man, x, K, N, th, tw, **kw):
    from comp_inference_amd import fused_rans_linear_triton

    dev = "cuda"
    return fused_rans_linear_triton(
        x.to(dev), torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
        torch.from_numpy(enc.slot_map).to(dev), (K, N), _t32(enc.tile_offsets).to(dev),
        _t32(enc.tile_max_lens).to(dev), th, tw, torch.from_numpy(man).to(dev), **kw)


@pytest.mark.parametrize("M", [1, 4, 16, 33, 64, 100])
@pytest.mark.parametrize("K,N,th,tw", [(4096, 256, 1024, 32), (3072, 128, 512, 32)])
def test_fused_linear_fast_path(oracle, M, K, N, th, tw):
    w = make_weight_kn(N, K, seed=1)
    enc, man, wdec = _compress(oracle, w, th, tw)
    x = make_x(M, K, seed=2)
    got = _call(enc, man, x, K, N, th, tw).float().cpu()
    want = torch.matmul(x.float(), wdec.float())
    assert got.shape == (M, N)
    assert torch.allclose(got, want, atol=ATOL, rtol=RTOL), (got - want).abs().max()


@pytest.mark.parametrize("K,N,th,tw,M", [
    (14336, 64, 1024, 32, 1),    # 14 k-tiles: two partial sums + reduction kernel
    (14336, 64, 1024, 32, 5),
    (14336, 64, 1024, 32, 40),   # two 32-row groups per pass + reduction kernel
    (1300, 80, 1024, 32, 50),    # two 32-row groups on the guarded path
    (1300, 80, 1024, 32, 3),     # ragged K and N
    (1000, 70, 512, 32, 2),
    (9000, 32, 1024, 32, 1),
    (2048, 32800, 1024, 32, 3),  # more tiles than the chip holds at once: resident workgroups, a partial per k-tile
    (2048, 32800, 1024, 32, 40),
    (256, 128, 64, 16, 4),       # other tile widths: generic kernel
    (384, 256, 128, 64, 9),
    (256, 256, 256, 128, 1),
])
def test_fused_linear_shapes(oracle, K, N, th, tw, M):
    w = make_weight_kn(N, K, seed=K + N)
    enc, man, wdec = _compress(oracle, w, th, tw)
    x = make_x(M, K, seed=M)
    got = _call(enc, man, x, K, N, th, tw).float().cpu()
    want = torch.matmul(x.float(), wdec.float())
    assert torch.allclose(got, want, atol=ATOL, rtol=RTOL), (got - want).abs().max()


def test_fused_linear_bias_out_and_batch_shape(oracle):
    K, N, th, tw = 2048, 96, 1024, 32
    w = make_weight_kn(N, K, seed=9)
    enc, man, wdec = _compress(oracle, w, th, tw)
    x = make_x(6, K, seed=3).view(2, 3, K)
    bias = make_x(1, N, seed=4).view(N)
    got = _call(enc, man, x, K, N, th, tw, bias=bias.cuda())
    assert got.shape == (2, 3, N) and got.dtype == torch.bfloat16
    want = (torch.matmul(x.float(), wdec.float()).to(torch.bfloat16) + bias).float()
    assert torch.allclose(got.float().cpu(), want, atol=ATOL, rtol=RTOL)
    out = torch.zeros(6, N, dtype=torch.bfloat16, device="cuda")
    ret = _call(enc, man, x, K, N, th, tw, bias=bias.cuda(), out=out)
    assert ret is out
    assert torch.equal(out.view(2, 3, N), got)


def test_fused_linear_is_deterministic(oracle):
    K, N, th, tw = 14336, 64, 1024, 32
    w = make_weight_kn(N, K, seed=21)
    enc, man, _ = _compress(oracle, w, th, tw)
    x = make_x(1, K, seed=22)
    a = _call(enc, man, x, K, N, th, tw)
    b = _call(enc, man, x, K, N, th, tw)
    assert torch.equal(a, b)


@pytest.mark.parametrize("K,N,th,tw,M", [(1024, 64, 512, 32, 3), (1024, 96, 1024, 32, 1), (700, 64, 1024, 32, 9),
                                         (1024, 4096, 1024, 32, 64), (256, 128, 256, 64, 5)])
def test_fused_linear_dense_layout(oracle, K, N, th, tw, M):
    """One stream per column and tile; with K <= tile_height there is a single partial sum per output,
    which still goes through the workspace and the reduction kernel."""
    from comp_inference_amd import fused_rans_linear_triton_uncoalesced

    w = make_weight_kn(N, K, seed=31)
    e, m = oracle.split_bf16(bf16_bits(w))
    f, c = oracle.get_lut(e)
    enc = oracle.encode_tiled_dense(e, f, c, th, tw)
    man = oracle.interleave_plane(m, th, tw)
    x = make_x(M, K, seed=32)
    dev = "cuda"
    got = fused_rans_linear_triton_uncoalesced(
        x.to(dev), torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
        torch.from_numpy(enc.slot_map).to(dev), (K, N), _t32(enc.stream_offsets).to(dev), _t32(enc.sizes).to(dev),
        th, tw, torch.from_numpy(man).to(dev))
    want = torch.matmul(x.float(), w.float())
    assert torch.allclose(got.float().cpu(), want, atol=ATOL, rtol=RTOL)


def test_splitk_reduce_matches_torch_sum():
    from comp_inference_amd import splitk_reduce

    g = torch.Generator("cpu").manual_seed(0)
    ws = torch.randn(8, 5, 96, generator=g).to(torch.bfloat16).cuda()
    bias = torch.randn(96, generator=g).to(torch.bfloat16).cuda()
    want = torch.sum(ws, dim=0)
    want += bias
    got = splitk_reduce(ws, bias=bias)
    assert torch.equal(got, want)


@pytest.mark.parametrize("P,M,N", [(128, 1, 128256), (14, 3, 40000), (5, 2, 32772), (9, 1, 70001)])
def test_splitk_reduce_fp32_both_kernels_sum_in_index_order(P, M, N):
    """fp32 partials (the library's own workspace layout): large outputs take the four-per-thread kernel,
    a workspace that is not 16-byte aligned (or a row length that is no multiple of 4) the one-per-thread
    kernel.  Both add plane after plane in index order, so they agree bit for bit with each other and
    with that loop written in torch."""
    import ctypes as C

    from comp_inference_amd import _lib

    g = torch.Generator("cpu").manual_seed(P + N)
    flat = torch.zeros(P * M * N + 4, dtype=torch.float32, device="cuda")
    data = torch.randn(P, M, N, generator=g).cuda()
    bias = torch.randn(N, generator=g).to(torch.bfloat16).cuda()
    want = torch.zeros(M, N, dtype=torch.float32, device="cuda")
    for p in range(P):
        want += data[p]
    want = want.to(torch.bfloat16)                       # rounded once, then the reference's bf16 `out += bias`
    want += bias

    def run(offset):
        part = flat[offset:offset + P * M * N]
        part.copy_(data.view(-1))
        assert part.data_ptr() % 16 == (0 if offset % 4 == 0 else 4 * (offset % 4))
        out = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
        rc = _lib.lib().ci_splitk_reduce(C.c_void_p(part.data_ptr()), 0, P, M, N, C.c_void_p(bias.data_ptr()),
                                         C.c_void_p(out.data_ptr()), N, _lib.stream_handle(out.device))
        assert rc == 0
        return out

    a, b = run(0), run(1)
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    assert torch.equal(a.view(torch.int16), want.view(torch.int16))


def test_dense_matmul_helper():
    """The uncompressed helper the reference exports as triton_matmul: shapes and tolerance."""
    from comp_inference_amd import triton_matmul

    b = make_weight_kn(96, 512, seed=3).cuda()           # [K=512, N=96]
    for shape in ((512,), (1, 512), (2, 3, 512)):
        a = make_x(int(np.prod(shape[:-1])) if len(shape) > 1 else 1, 512, seed=len(shape)).view(*shape).cuda()
        got = triton_matmul(a, b)
        assert got.dtype == torch.bfloat16 and tuple(got.shape) == (*shape[:-1], 96)
        want = torch.matmul(a.float().view(-1, 512), b.float()).view(*shape[:-1], 96)
        assert torch.allclose(got.float(), want, atol=ATOL, rtol=RTOL)
    with pytest.raises(RuntimeError):
        triton_matmul(torch.zeros(1, 512, dtype=torch.bfloat16), b)


@pytest.mark.parametrize("K,N,th,M", [
    (4096, 256, 1024, 1), (4096, 256, 1024, 16), (4096, 256, 1024, 17), (4096, 256, 1024, 64),
    (4096, 256, 1024, 100),      # more than 64 rows: one pass per 64
    (3072, 128, 512, 4),
    (14336, 64, 1024, 1),        # two partial sums per output + reduction kernel
    (14336, 64, 1024, 40),
    (1300, 80, 1024, 3),         # ragged K and N: guarded path in both runs
    (1300, 80, 1024, 50),
    (2048, 32800, 1024, 3),      # resident workgroups, one partial per k-tile
    (2048, 32800, 1024, 40),
])
def test_fused_linear_bit_identical_to_plain_weight_contraction(oracle, K, N, th, M):
    """The fused kernel on the compressed weight and the same contraction on the plain bf16 weight give
    the same bits: every weight bit, sign and low mantissa bits included, reaches the matrix unit
    as the encoder saw it -- which the 1e-2 tolerance against torch.matmul cannot show."""
    from comp_inference_amd import plain_linear_same_order

    w = make_weight_kn(N, K, seed=K + N + 1)
    enc, man, wdec = _compress(oracle, w, th, 32)
    x = make_x(M, K, seed=M + 7)
    bias = make_x(1, N, seed=3).view(N) if M == 3 else None
    got = _call(enc, man, x, K, N, th, 32, bias=bias)
    same = plain_linear_same_order(x.cuda(), wdec.cuda(), tile_k=th, tile_n=32,
                                   bias=None if bias is None else bias.cuda())
    assert same.shape == got.shape and same.dtype == torch.bfloat16
    assert torch.equal(got.view(torch.int16), same.view(torch.int16))
    want = torch.matmul(x.float(), wdec.float()) + (0 if bias is None else bias.float())
    assert torch.allclose(same.float().cpu(), want, atol=ATOL, rtol=RTOL)


@pytest.mark.parametrize("K,N,M,P", [(14336, 64, 1, 2), (14336, 64, 40, 2), (2048, 32800, 3, 2)])
def test_fp32_partial_sums_bit_identical_and_sharp(oracle, K, N, M, P):
    """Where the contraction is split over K the fp32 partial sums stay in the caller's workspace: they
    too are equal bit for bit, and one flipped low mantissa bit of one weight changes exactly the
    partial sums of its column -- an error far below what the bf16 output or a 1e-2 tolerance shows."""
    from comp_inference_amd import plain_linear_same_order

    th = 1024
    w = make_weight_kn(N, K, seed=K + N + 2)
    enc, man, wdec = _compress(oracle, w, th, 32)
    x = make_x(M, K, seed=M + 30)
    nbytes = P * M * N * 4 + (1 << 22)
    ws_a = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    ws_b = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    got = _call(enc, man, x, K, N, th, 32, workspace=ws_a)
    same = plain_linear_same_order(x.cuda(), wdec.cuda(), tile_k=th, tile_n=32, workspace=ws_b)
    pa = ws_a[:P * M * N * 4].view(torch.int32).view(P, M, N)
    pb = ws_b[:P * M * N * 4].view(torch.int32).view(P, M, N)
    assert torch.equal(got.view(torch.int16), same.view(torch.int16))
    assert torch.equal(pa, pb)
    assert int((pa != 0).sum()) > P * M * N // 2       # (the workspace really holds the partial sums)

    bits = wdec.view(torch.int16).clone()
    k = int(x[0].float().abs().argmax())               # a row of the weight that certainly contributes
    bits[k, 5] ^= 1
    plain_linear_same_order(x.cuda(), bits.view(torch.bfloat16).cuda(), tile_k=th, tile_n=32, workspace=ws_b)
    torch.cuda.synchronize()
    diff = (pa != pb).nonzero()
    assert diff.numel() > 0 and set(diff[:, 2].tolist()) == {5}


def test_plain_weight_contraction_rejects_other_tilings():
    from comp_inference_amd import plain_linear_same_order

    x = torch.zeros(1, 256, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(256, 128, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError):
        plain_linear_same_order(x, w, tile_k=64, tile_n=16)
    with pytest.raises(RuntimeError):
        plain_linear_same_order(x.cpu(), w)


def test_many_rows_decode_the_weight_once(oracle):
    """Above DECODE_ONCE_ABOVE_ROWS rows the weight is decoded once and a library GEMM does the product:
    the result is torch.matmul on the decoded weight, bit for bit, with bias and a strided `out`."""
    from comp_inference_amd import linear_hip

    K, N, th, M = 2048, 160, 1024, 200
    assert M > linear_hip.DECODE_ONCE_ABOVE_ROWS
    w = make_weight_kn(N, K, seed=21)
    enc, man, wdec = _compress(oracle, w, th, 32)
    x = make_x(M, K, seed=22).cuda()
    bias = make_x(1, N, seed=23).view(N).cuda()
    want = torch.matmul(x, wdec.cuda())
    want += bias
    got = _call(enc, man, x, K, N, th, 32, bias=bias)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    big = torch.zeros(M, N + 32, dtype=torch.bfloat16, device="cuda")
    ret = _call(enc, man, x, K, N, th, 32, bias=bias, out=big[:, :N])
    assert ret.data_ptr() == big.data_ptr()
    assert torch.equal(big[:, :N].view(torch.int16), want.view(torch.int16)) and not big[:, N:].any()
    # 3-D input keeps its leading shape
    got3 = _call(enc, man, x.view(2, 100, K), K, N, th, 32)
    assert tuple(got3.shape) == (2, 100, N)
    # with decoder checkpoints the one decode runs segmented: same weight, same product
    from comp_inference_amd import build_checkpoints

    ck = build_checkpoints(torch.from_numpy(enc.stream).cuda(), _t32(enc.states).cuda(), _t32(enc.tables).cuda(),
                           torch.from_numpy(enc.slot_map).cuda(), (K, N), _t32(enc.tile_offsets).cuda(),
                           _t32(enc.tile_max_lens).cuda(), th, 32, 4)
    got4 = _call(enc, man, x, K, N, th, 32, bias=bias, checkpoints=ck, segments=4)
    assert torch.equal(got4.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("K,N,th,M", [(4096, 256, 1024, 100), (3072, 128, 512, 150), (1300, 80, 1024, 70)])
def test_fused_kernels_above_64_rows(oracle, always_fused, K, N, th, M):
    """With the decode-once policy off, more than 64 rows run the fused kernel in passes of 64: within
    tolerance of torch.matmul and bit-identical to the same contraction on the plain weight."""
    from comp_inference_amd import plain_linear_same_order

    w = make_weight_kn(N, K, seed=K + M)
    enc, man, wdec = _compress(oracle, w, th, 32)
    x = make_x(M, K, seed=M)
    got = _call(enc, man, x, K, N, th, 32)
    want = torch.matmul(x.float(), wdec.float())
    assert torch.allclose(got.float().cpu(), want, atol=ATOL, rtol=RTOL), (got.float().cpu() - want).abs().max()
    same = plain_linear_same_order(x.cuda(), wdec.cuda(), tile_k=th, tile_n=32)
    assert torch.equal(got.view(torch.int16), same.view(torch.int16))
    # and it is not the library GEMM's summation order
    assert not torch.equal(got.view(torch.int16), torch.matmul(x.cuda(), wdec.cuda()).view(torch.int16))


def test_fused_linear_random_shapes(oracle, always_fused):
    """Thirty seeded random shapes (ragged K and N, 1 to 70 rows of x, three tile heights) on the fused
    kernels: within tolerance of torch.matmul and bit-identical to the plain-weight contraction."""
    from comp_inference_amd import plain_linear_same_order

    rng = np.random.default_rng(77)
    for case in range(30):
        th = int(rng.choice([64, 256, 1024]))
        K = int(rng.integers(1, 3 * th + 1))
        N = int(rng.integers(8, 200))   # (fewer real columns than 8 of 32 overrun the reference's stream capacity)
        M = int(rng.integers(1, 71))
        w = make_weight_kn(N, K, seed=2000 + case)
        enc, man, wdec = _compress(oracle, w, th, 32)
        x = make_x(M, K, seed=3000 + case)
        got = _call(enc, man, x, K, N, th, 32)
        want = torch.matmul(x.float(), wdec.float())
        assert torch.allclose(got.float().cpu(), want, atol=ATOL, rtol=RTOL), (case, K, N, M, th)
        same = plain_linear_same_order(x.cuda(), wdec.cuda(), tile_k=th, tile_n=32)
        assert torch.equal(got.view(torch.int16), same.view(torch.int16)), (case, K, N, M, th)


def _pyref_resume(enc, ck, tile, q, seg, seglen, th):
    """Symbols of segment `seg` of stream q of `tile`, decoded from its checkpoint with plain integers."""
    spt = 64
    tables, slot_map = enc.tables, enc.slot_map
    x, row = (int(enc.states[tile * spt + q]), int(enc.tile_max_lens[tile]) - 1) if seg == 0 else \
        (int(ck[tile, seg - 1, q]) & 0xFFFFFFFF, ((int(ck[tile, seg - 1, q]) >> 32) + (1 << 31)) % (1 << 32) - (1 << 31))
    base, out = int(enc.tile_offsets[tile]), []
    for _ in range(seglen):
        slot = x & 4095
        s = int(slot_map[slot])
        out.append(s)
        f, c = int(tables[s]) & 0xFFFF, int(tables[s]) >> 16
        x = f * (x >> 12) + slot - c
        for _ in range(2):
            if x < (1 << 16) and row >= 0:
                x = (x << 8) | int(enc.stream[base + row * spt + q])
                row -= 1
    return out, x, row


@pytest.mark.parametrize("segments", [2, 4, 8])
def test_checkpoints_resume_the_decoder(oracle, segments):
    """A checkpoint is the decoder's state and byte position at the first row of a segment: decoding on from
    it gives that segment's symbols and arrives exactly at the next checkpoint."""
    from comp_inference_amd import build_checkpoints

    K, N, th = 2048, 64, 1024
    w = make_weight_kn(N, K, seed=61)
    enc, man, wdec = _compress(oracle, w, th, 32)
    exp_plane = (bf16_bits(wdec) >> 7).astype(np.uint8)
    dev = "cuda"
    ck = build_checkpoints(torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
                           torch.from_numpy(enc.slot_map).to(dev), (K, N), _t32(enc.tile_offsets).to(dev),
                           _t32(enc.tile_max_lens).to(dev), th, 32, segments).cpu().numpy()
    assert ck.shape == (4, segments - 1, 64)
    half, seglen = th // 2, th // 2 // segments
    for tile, q in ((0, 0), (1, 37), (3, 63), (2, 5)):
        tk, tn = divmod(tile, 2)
        col, r0 = tn * 32 + q % 32, tk * th + (q // 32) * half
        for seg in range(segments):
            syms, x, row = _pyref_resume(enc, ck, tile, q, seg, seglen, th)
            assert syms == exp_plane[r0 + seg * seglen: r0 + (seg + 1) * seglen, col].tolist(), (tile, q, seg)
            if seg + 1 < segments:
                nxt = int(ck[tile, seg, q])
                assert (x, row) == (nxt & 0xFFFFFFFF, ((nxt >> 32) + (1 << 31)) % (1 << 32) - (1 << 31))
            else:
                assert x == 1 << 16  # the stream ends where the encoder began


@pytest.mark.parametrize("K,N,th,M,segments", [
    (4096, 256, 1024, 1, 2), (4096, 256, 1024, 1, 4), (4096, 256, 1024, 1, 8), (4096, 256, 1024, 16, 4),
    (4096, 256, 1024, 17, 4), (4096, 256, 1024, 64, 2),
    (3072, 128, 512, 4, 4),
    (1300, 80, 1024, 3, 4),     # ragged: short last tile row, 80 columns
    (1300, 80, 1024, 50, 2),
    (2048, 32800, 1024, 3, 2),  # many tiles and segments
])
def test_segmented_fused_linear(oracle, K, N, th, M, segments):
    """With decoder checkpoints every (tile, segment) is decoded by a wavefront of its own: same result
    within tolerance, and bit-identical to the plain-weight contraction split the same way."""
    from comp_inference_amd import build_checkpoints, plain_linear_same_order

    w = make_weight_kn(N, K, seed=K + N + segments)
    enc, man, wdec = _compress(oracle, w, th, 32)
    x = make_x(M, K, seed=M + segments)
    dev = "cuda"
    ck = build_checkpoints(torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
                           torch.from_numpy(enc.slot_map).to(dev), (K, N), _t32(enc.tile_offsets).to(dev),
                           _t32(enc.tile_max_lens).to(dev), th, 32, segments)
    bias = make_x(1, N, seed=5).view(N) if M == 3 else None
    got = _call(enc, man, x, K, N, th, 32, checkpoints=ck, segments=segments, bias=bias)
    want = torch.matmul(x.float(), wdec.float()) + (0 if bias is None else bias.float())
    assert torch.allclose(got.float().cpu(), want, atol=ATOL, rtol=RTOL), (got.float().cpu() - want).abs().max()
    same = plain_linear_same_order(x.cuda(), wdec.cuda(), tile_k=th, tile_n=32, segments=segments,
                                   bias=None if bias is None else bias.cuda())
    assert torch.equal(got.view(torch.int16), same.view(torch.int16))
    again = _call(enc, man, x, K, N, th, 32, checkpoints=ck, segments=segments, bias=bias)
    assert torch.equal(got, again)


def test_segment_arguments_are_checked(oracle):
    from comp_inference_amd import build_checkpoints, suggest_segments

    assert suggest_segments((4096, 4096)) == 8 and suggest_segments((4096, 14336)) == 2
    assert suggest_segments((4096, 28672)) == 2 and suggest_segments((4096, 4096), 1024, 64) == 1
    K, N, th = 1024, 64, 1024
    w = make_weight_kn(N, K, seed=71)
    enc, man, wdec = _compress(oracle, w, th, 32)
    dev = "cuda"
    args = (torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
            torch.from_numpy(enc.slot_map).to(dev), (K, N), _t32(enc.tile_offsets).to(dev), _t32(enc.tile_max_lens).to(dev))
    assert build_checkpoints(*args, th, 32, 1) is None
    with pytest.raises(RuntimeError):
        build_checkpoints(*args, th, 32, 3)            # 512 rows do not split into 3 equal segments
    ck = build_checkpoints(*args, th, 32, 4)
    x = make_x(2, K, seed=1)
    with pytest.raises(RuntimeError):
        _call(enc, man, x, K, N, th, 32, checkpoints=ck, segments=2)   # index made for 4 segments


def _window_rows_numpy(ck, depths, segments):
    """Rows of a tile body that item (tile, segment) can touch, from the checkpoint index alone: from the lowest
    row any lane has reached at the segment's end to the highest row a lane starts at; maximum over all items."""
    best = 1
    tiles = depths.shape[0]
    rows = None if ck is None else (ck >> 32).astype(np.int64)  # (int64 words: the shift keeps the row's sign)
    for t in range(tiles):
        d = int(depths[t])
        for seg in range(segments):
            start = np.full(64, d - 1, np.int64) if seg == 0 else np.minimum(rows[t, seg - 1], d - 1)
            end = np.minimum(rows[t, seg], start) if seg + 1 < segments else np.full(64, -1, np.int64)
            lo, hi = max(int(end.min()), 0), int(start.max())
            best = max(best, hi - lo + 1 if hi >= lo else 0)
    return best


@pytest.mark.parametrize("K,N,th,M,segments", [
    (4096, 256, 1024, 1, 2), (4096, 256, 1024, 5, 4), (4096, 256, 1024, 40, 8), (8192, 64, 1024, 1, 2),
    (18432, 64, 1024, 3, 2),  # 36 items per column tile: two chunks, partial sums through the workspace
    (2048, 96, 512, 1, 1),    # no checkpoints: whole streams of a 256-row half tile
])
def test_prepared_weight_runs_the_kernel_without_guarded_path(oracle, K, N, th, M, segments):
    """A prepared weight knows its largest window (ci_max_window_rows, checked here against the checkpoint
    index) and, on whole tiles, runs the kernel instance that has no guarded path: its output is the same bits
    as the checking instance's, which the operator without a prepared weight runs."""
    from comp_inference_amd import build_checkpoints
    from comp_inference_amd.linear_hip import PreparedLinear

    w = make_weight_kn(N, K, seed=K + N + segments)
    enc, man, wdec = _compress(oracle, w, th, 32)
    x = make_x(M, K, seed=M).cuda()
    dev = torch.device("cuda", 0)
    args = (torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
            torch.from_numpy(enc.slot_map).to(dev), (K, N), _t32(enc.tile_offsets).to(dev), _t32(enc.tile_max_lens).to(dev))
    ck = build_checkpoints(*args, th, 32, segments)
    p = PreparedLinear(dev, *args, th, 32, torch.from_numpy(man).to(dev), checkpoints=ck, segments=segments)
    want_rows = _window_rows_numpy(None if ck is None else ck.cpu().numpy(), enc.tile_max_lens.astype(np.int64), segments)
    assert p.max_window_rows == want_rows
    assert 0 < p.max_window_rows <= 112
    got = p(x)
    same = _call(enc, man, x, K, N, th, 32, checkpoints=ck, segments=segments)
    assert torch.equal(got.view(torch.int16), same.view(torch.int16))
    want = torch.matmul(x.float().cpu(), wdec.float())
    assert torch.allclose(got.float().cpu(), want, atol=ATOL, rtol=RTOL)


def test_a_window_promise_that_is_too_small_loses_items_but_stays_in_bounds(oracle):
    """Exponents spread evenly over sixteen values cost half a byte per symbol, so a 256-row half tile reads
    more rows of its body than an item's staging area holds.  With no promise in the descriptor the checking
    kernel sends such items down the guarded path and the result is right; with a promise that is too small the
    kernel without guarded path leaves them out: wrong sums, but nothing out of bounds, and the next call is
    unharmed."""
    import ctypes as C

    from comp_inference_amd import _lib

    K, N, th = 1024, 64, 512
    rng = np.random.default_rng(17)
    bits = (rng.integers(0, 2, (K, N)) << 15 | rng.integers(118, 134, (K, N)) << 7 | rng.integers(0, 128, (K, N))).astype(np.uint16)
    w = bits_to_bf16(bits)
    enc, man, wdec = _compress(oracle, w, th, 32)
    dev = torch.device("cuda", 0)
    t = [torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
         torch.from_numpy(enc.slot_map).to(dev), _t32(enc.tile_offsets).to(dev), _t32(enc.tile_max_lens).to(dev),
         torch.from_numpy(man).to(dev)]
    x = make_x(2, K, seed=3).to(dev)
    lib, ptr = _lib.lib(), _lib.ptr
    need = lib.ci_fused_linear_workspace_bytes_segmented(2, K, N, th, 32, 0, 1)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)

    def run(promise):
        desc = _lib.tiled_weight(K, N, th, 32, t[0], t[1], t[2], t[3], t[4], t[5], t[6], None, 1, None, promise)
        out = torch.zeros(2, N, dtype=torch.bfloat16, device=dev)
        _lib.check(lib.ci_fused_linear_tiled(C.byref(desc), ptr(x), 2, K, None, ptr(out), N, ptr(ws), C.c_size_t(ws.numel()),
                                             _lib.stream_handle(dev)))
        torch.cuda.synchronize()
        return out.float().cpu()

    rows = torch.zeros(1, dtype=torch.int32, device=dev)
    desc = _lib.tiled_weight(K, N, th, 32, t[0], t[1], t[2], t[3], t[4], t[5], t[6])
    _lib.check(lib.ci_max_window_rows(C.byref(desc), ptr(rows), _lib.stream_handle(dev)))
    true_rows = int(rows.item())
    assert true_rows == int(enc.tile_max_lens.max()) and true_rows > 112
    want = torch.matmul(x.float().cpu(), wdec.float())
    right = run(0)
    assert torch.allclose(right, want, atol=ATOL, rtol=RTOL)
    assert torch.equal(run(true_rows), right)   # the true figure is beyond the staging area: the checking kernel again
    lost = run(100)
    assert bool(torch.isfinite(lost).all()) and not torch.equal(lost, right)
    assert torch.equal(run(0), right)
