"""The sixteen-wavefront LM-head kernel (one row of x, decoder checkpoints, largest window known) against the
kernel that walks whole tiles: the same products and the same eight-row reduction, so the logits are compared bit
for bit; and against torch.matmul on the oracle-decoded weight within the operator's tolerance."""
import ctypes as C

import numpy as np
import pytest
import torch

from helpers import bf16_bits, bits_to_bf16, make_weight_kn, make_x

pytestmark = pytest.mark.gpu
ATOL = RTOL = 1e-2


def _t32(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int32))


@pytest.mark.parametrize("V,H,segments", [(2304, 128, 2), (4096, 64, 4), (1024, 96, 2), (3000, 64, 2)])
def test_one_row_of_x_on_sixteen_wavefronts(oracle, V, H, segments):
    import comp_inference_amd as ci
    from comp_inference_amd import _lib

    th = 1024
    w = make_weight_kn(H, V, seed=V + H)           # [V, H]: rows are the outputs
    enc, man = oracle.compress_bf16(bf16_bits(w), th, 32)
    wdec = bits_to_bf16(oracle.decompress_bf16(enc, man, V, H))
    dev = torch.device("cuda", 0)
    t = [torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
         torch.from_numpy(enc.slot_map).to(dev), _t32(enc.tile_offsets).to(dev), _t32(enc.tile_max_lens).to(dev),
         torch.from_numpy(man).to(dev)]
    args = (t[0], t[1], t[2], t[3], (V, H), t[4], t[5], th, 32, t[6])
    x = make_x(1, H, seed=7).to(dev)
    whole = ci.fused_rans_linear_transposed(x, *args)
    ck = ci.build_checkpoints(t[0], t[1], t[2], t[3], (V, H), t[4], t[5], th, 32, segments)
    rows = torch.zeros(1, dtype=torch.int32, device=dev)
    desc = _lib.tiled_weight(V, H, th, 32, t[0], t[1], t[2], t[3], t[4], t[5], None, ck, segments)
    _lib.check(_lib.lib().ci_max_window_rows(C.byref(desc), _lib.ptr(rows), _lib.stream_handle(dev)))
    max_rows = int(rows.item())
    assert 0 < max_rows <= 112
    got = ci.fused_rans_linear_transposed(x, *args, checkpoints=ck, segments=segments, max_window_rows=max_rows)
    assert torch.equal(got.view(torch.int16), whole.view(torch.int16))
    want = torch.matmul(x.float().cpu(), wdec.float().t())
    assert torch.allclose(got.float().cpu(), want, atol=ATOL, rtol=RTOL), (got.float().cpu() - want).abs().max()
    # more rows of x, or no promise about the windows, take the other kernel: same answer as without checkpoints
    x3 = make_x(3, H, seed=8).to(dev)
    assert torch.equal(ci.fused_rans_linear_transposed(x3, *args, checkpoints=ck, segments=segments, max_window_rows=max_rows),
                       ci.fused_rans_linear_transposed(x3, *args))
    assert torch.equal(ci.fused_rans_linear_transposed(x, *args, checkpoints=ck, segments=segments), whole)


def test_tile_bodies_without_a_byte(oracle):
    """A constant exponent plane in low tiles: no stream emits a byte, every body has depth 0 and every window is
    empty; the items are decoded all the same (their rows once surfaced as whatever the workspace held)."""
    import comp_inference_amd as ci

    V, H, th, segments = 384, 64, 128, 2
    g = torch.Generator("cpu").manual_seed(1)
    w = ((1.0 + torch.rand(V, H, generator=g) * 0.99) * torch.where(torch.rand(V, H, generator=g) < 0.5, -1.0, 1.0)).to(torch.bfloat16)
    enc, man = oracle.compress_bf16(bf16_bits(w), th, 32)
    assert not enc.tile_max_lens.any()
    dev = torch.device("cuda", 0)
    t = [torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
         torch.from_numpy(enc.slot_map).to(dev), _t32(enc.tile_offsets).to(dev), _t32(enc.tile_max_lens).to(dev),
         torch.from_numpy(man).to(dev)]
    args = (t[0], t[1], t[2], t[3], (V, H), t[4], t[5], th, 32, t[6])
    x = make_x(1, H, seed=7).to(dev)
    whole = ci.fused_rans_linear_transposed(x, *args)
    ck = ci.build_checkpoints(t[0], t[1], t[2], t[3], (V, H), t[4], t[5], th, 32, segments)
    torch.full((1 << 20,), float("nan"), device=dev)  # (what a recycled workspace may hold)
    got = ci.fused_rans_linear_transposed(x, *args, checkpoints=ck, segments=segments, max_window_rows=1)
    assert torch.equal(got.view(torch.int16), whole.view(torch.int16))
    assert torch.allclose(got.float().cpu(), x.float().cpu() @ w.float().t(), atol=ATOL, rtol=RTOL)


def test_the_module_takes_the_kernel_when_segments_are_switched_on():
    import comp_inference_amd as ci

    V, H = 4096, 128
    emb = torch.nn.Embedding(V, H).to(torch.bfloat16)
    table = emb.weight.detach().clone()
    ci.rans_compress_module_weight(emb, tile_height=1024, tile_width=32, transpose_weight=False)
    re = ci.RansEmbedding.from_compressed(emb)
    head = ci.RansLMHead(H, V)
    head.tie_to(re)
    h = make_x(1, H, seed=3)
    whole = head(h.cuda())
    assert torch.allclose(whole.float().cpu(), h.float() @ table.float().t(), atol=ATOL, rtol=RTOL)
    head.segments = "auto"
    ck, segs, max_rows, slot_table = head._derived(torch.device("cuda", 0))
    assert segs > 1 and 0 < max_rows <= 112 and slot_table.numel() == 32768
    assert torch.equal(head(h.cuda()), whole)
    h3 = make_x(3, H, seed=4)
    head.segments = 1
    whole3 = head(h3.cuda())
    head.segments = "auto"
    assert torch.equal(head(h3.cuda()), whole3)


@pytest.mark.parametrize("V,H,segments", [(2304, 128, 2), (4096, 64, 4), (1024, 96, 8), (8192, 256, 2)])
def test_sums_on_the_matrix_pipe(oracle, V, H, segments):
    """`head_matrix_sums`: another order of the sum over the hidden dimension, so the bar is the operator's tolerance
    against torch.matmul, a tight bound against the float64 product (every output is 16 + 16 fp32 multiply-adds of
    exact bf16 products), the same bits on a second call, and the other kernel's answer back once switched off."""
    import comp_inference_amd as ci
    from comp_inference_amd import _lib

    th = 1024
    w = make_weight_kn(H, V, seed=V + H + 1)
    enc, man = oracle.compress_bf16(bf16_bits(w), th, 32)
    dev = torch.device("cuda", 0)
    t = [torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
         torch.from_numpy(enc.slot_map).to(dev), _t32(enc.tile_offsets).to(dev), _t32(enc.tile_max_lens).to(dev),
         torch.from_numpy(man).to(dev)]
    args = (t[0], t[1], t[2], t[3], (V, H), t[4], t[5], th, 32, t[6])
    x = make_x(1, H, seed=9).to(dev)
    ck = ci.build_checkpoints(t[0], t[1], t[2], t[3], (V, H), t[4], t[5], th, 32, segments)
    rows = torch.zeros(1, dtype=torch.int32, device=dev)
    desc = _lib.tiled_weight(V, H, th, 32, t[0], t[1], t[2], t[3], t[4], t[5], None, ck, segments)
    _lib.check(_lib.lib().ci_max_window_rows(C.byref(desc), _lib.ptr(rows), _lib.stream_handle(dev)))
    kw = dict(checkpoints=ck, segments=segments, max_window_rows=int(rows.item()))
    lanes = ci.fused_rans_linear_transposed(x, *args, **kw)
    assert ci.head_matrix_sums(True) is False
    try:
        got = ci.fused_rans_linear_transposed(x, *args, **kw)
        again = ci.fused_rans_linear_transposed(x, *args, **kw)
    finally:
        assert ci.head_matrix_sums(False) is True
    assert torch.equal(got, again)
    want64 = (x.double().cpu() @ w.double().t())
    assert torch.allclose(got.float().cpu(), want64.float(), atol=ATOL, rtol=RTOL)
    # fp32 sums of at most H exact products, rounded once to bf16: within a bf16 step of the exact value
    scale = (x.double().cpu().abs() @ w.double().abs().t())
    assert ((got.double().cpu() - want64).abs() <= scale * 2.0 ** -8 + 1e-30).all()
    assert torch.equal(ci.fused_rans_linear_transposed(x, *args, **kw), lanes)
