"""The benchmark configurations' shapes on the host model (tests/hostmodel), at the sizes the CPU model can run in a
minute: the Llama-3-8B gate projection (4096 x 14336, tile 1024 x 32, bf16 N(0, 0.02)) whole, the k projection, and
the 128,256-row embedding table with a sixteenth of its columns (column tiles are independent work items: the row
count is what shapes buckets, chunks and checkpoints).  Same checks as the other test_hostmodel_* files: results
against the oracle, every address against the arrays, 256 CUs as on the chip."""
import numpy as np

from tests.hostmodel import cases
from tests.hostmodel.model import Model, in_fresh_process, weight_bits, x_bits

CUS = 256


@in_fresh_process
def test_gate_projection_decode_and_gemv_at_full_size():
    """Configurations 1 and 2: the gate projection decoded in one launch (decoder checkpoints at the middle of every
    stream, as bench.py runs it) and the fused GEMV for one row of x on the prepared weight."""
    import ctypes as C

    from oracle import rans_oracle as ro

    m = Model(cus=CUS)
    K, N, th = 4096, 14336, 1024
    bits = weight_bits(K, N, 1)
    enc, man = cases.compress(bits, th)
    w, keep = m.weight(enc, man, K, N, segments=2, slot_table=True, window_rows=True)
    assert 2 <= w.max_window_rows <= 112, w.max_window_rows
    out = m.empty((K, N), np.uint8)
    m.clear()
    m.call("ci_decode_tiled", C.byref(w), out.p, None, None)
    assert m.launches() == ["decode_tiled32_seg_kernel<false>"]
    assert np.array_equal(out.get(), ro.split_bf16(bits)[0])
    xb = x_bits(1, K, 2)
    x, y = m.dev(xb), m.empty((1, N), np.uint16)
    nb = m.lib.ci_fused_linear_workspace_bytes_segmented(1, K, N, th, 32, 0, 2)
    ws = m.empty(max(nb, 16), np.uint8)
    m.clear()
    m.call("ci_fused_linear_tiled", C.byref(w), x.p, 1, K, None, y.p, N, ws.p, C.c_size_t(nb), None)
    assert m.launches() == ["(fused_linear32_seg_kernel<1, false>)"], m.launches()
    want = ro.linear_f32(xb, bits)
    from tests.hostmodel.model import bf16_bits_to_f32

    assert np.allclose(bf16_bits_to_f32(y.get()), want, atol=1e-2, rtol=1e-2)


@in_fresh_process
def test_k_projection_every_operator():
    """1024 x 4096 stored [K = 4096, N = 1024]: decode with and without checkpoints, GEMV / GEMM at the rows of
    configuration 2 and above 64 rows."""
    m = Model(cus=CUS)
    bits = weight_bits(4096, 1024, 1)
    cases.decode(m, bits, 1024, 1, expect_kernel="decode_tiled32_persist_kernel<false>")
    cases.decode(m, bits, 1024, 2, merge=True, expect_kernel="decode_tiled32_seg_kernel<true>")
    for M, segs in ((1, 4), (4, 4), (16, 4), (64, 4)):
        cases.linear(m, bits, x_bits(M, 4096, 2), 1024, segs, slot_table=True, window_rows=True,
                     expect_kernel="fused_linear32_seg_kernel")
    cases.linear(m, bits, x_bits(128, 4096, 2), 1024, wide=True, expect_kernel="fused_linear32_wide_kernel<4>")


@in_fresh_process
def test_embedding_table_rows_gather_and_lm_head():
    """Configuration 3's 128,256 rows (last tile row 256 rows: its bottom-half streams are empty) and 2048 Zipf(1.1)
    ids from numpy's default_rng(4), on 256 of the 4096 columns: the gather with 8 segments per stream through the
    sixteen-wavefront kernel and through the twelve-wavefront one, then the table's first 16 tile rows as an LM head
    for one row of x with both kinds of sums."""
    m = Model(cus=CUS)
    V, H, th = 128256, 256, 1024
    bits = weight_bits(V, H, 3)
    rng = np.random.default_rng(4)
    p = 1.0 / np.arange(1, V + 1) ** 1.1
    ids = rng.choice(V, 2048, p=p / p.sum()).astype(np.int64)
    cases.gather(m, bits, ids, th, 8, slot_table=True, expect_kernel="embed_gather32_seg_kernel")
    cases.gather(m, bits, ids, th, 8, slot_table=False, expect_kernel="embed_gather32_kernel")
    m.free_all()
    head = np.ascontiguousarray(bits[:16 * th + 256])
    cases.lm_head(m, head, x_bits(1, H, 2), th, 2, window_rows=True, expect_kernel="trans32_seg_kernel<false>")
    cases.lm_head(m, head, x_bits(1, H, 2), th, 2, window_rows=True, slot_table=True, matrix_sums=True, check_twin=False,
                  expect_kernel="trans32_seg_kernel<true>")
