"""Every kernel of the library on the host model (tests/hostmodel): the library's own sources compiled for the CPU,
the assembly statements interpreted, every address the interpreter forms checked against the exact extent of the
arrays and every array ending at an inaccessible page.  Results are compared with the oracle (bit-exact decode,
encode and gather; fused linears within 1e-2 of the fp32 product and bit for bit with the same contraction on the
plain weight), and each case names the kernel it must have run.

The kernels that have run on the GPU (decode, the fused linear's plans, the gather, the LM head) give the oracle's
results here too, which is what ties the model to the hardware; the kernels that have not yet run on a GPU
(embed_gather32_seg_kernel, fused_linear32_wide_kernel, trans32_seg_kernel with both kinds of sums, the entry points of
the one-stream-per-column layout) are held to the same checks before their first launch."""
import numpy as np
import pytest

from tests.hostmodel import cases
from tests.hostmodel.model import Model, in_child, weight_bits, x_bits


# ---- stand-alone decode -----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("K,N,th,segs,merge,kernel", [
    (2048, 128, 1024, 1, False, "decode_tiled32_persist_kernel<false>"),
    (2048, 128, 1024, 1, True, "decode_tiled32_persist_kernel<true>"),
    (2048, 128, 1024, 2, False, "decode_tiled32_seg_kernel<false>"),
    (2048, 128, 1024, 4, True, "decode_tiled32_seg_kernel<true>"),
    (1024, 96, 512, 1, False, "decode_tiled32_seg_kernel<false>"),   # low tiles: whole streams on sixteen wavefronts
    (2048 + 300, 100, 1024, 2, False, "decode_tiled32_seg_kernel<false>"),  # ragged rows and columns, odd last tile
    (3000, 70, 2048, 1, True, "decode_tiled32_persist_kernel<true>"),
    (2048, 95, 1024, 2, False, "decode_tiled32_seg_kernel<false>"),   # one column short of whole tiles: the 64-byte rows of a pair end one byte early
    (1024, 63, 1024, 1, False, "decode_tiled32_persist_kernel<false>"),
    (2048, 63, 1024, 2, False, "decode_tiled32_seg_kernel<false>"),   # ... of a whole pair of tiles
    (2048, 127, 1024, 4, True, "decode_tiled32_seg_kernel<true>"),
    (512, 63, 256, 2, False, "decode_tiled32_seg_kernel<false>"),     # ... with short items, whose last one ends the array
    (768, 127, 256, 1, False, "decode_tiled32_seg_kernel<false>"),
])
@in_child
def test_decode(K, N, th, segs, merge, kernel):
    cases.decode(Model(cus=4), weight_bits(K, N, 1), th, segs, merge, expect_kernel=kernel)


@pytest.mark.parametrize("kind", cases.KINDS)
@in_child
def test_decode_of_unusual_planes(kind):
    rng = np.random.default_rng(11)
    for segs in (1, 2, 8):
        cases.decode(Model(cus=3), cases.weight_kind(rng, 2048, 96, kind), 1024, segs)


@in_child
def test_decode_batch_of_a_layer_in_one_launch():
    """ci_decode_tiled_ilp2_batch: several tensors, with and without checkpoints, CUs divided among them."""
    import ctypes as C

    from oracle import rans_oracle as ro
    from tests.hostmodel.model import DecodeItem

    m = Model(cus=6)
    shapes = [(1024, 128, 1), (2048, 64, 2), (1024, 256, 4), (1500, 40, 2)]
    items = (DecodeItem * len(shapes))()
    keep, outs, refs = [], [], []
    for i, (K, N, segs) in enumerate(shapes):
        bits = weight_bits(K, N, 20 + i)
        enc, man = cases.compress(bits, 1024)
        w, kp = m.weight(enc, None, K, N, segments=segs)
        out = m.empty((K, N), np.uint8)
        keep.append((w, kp))
        outs.append(out)
        refs.append(ro.split_bf16(bits)[0])
        it = items[i]
        it.d_stream, it.stream_len, it.d_states, it.d_tables, it.d_slot_map = w.d_stream, w.stream_len, w.d_states, w.d_tables, w.d_slot_map
        it.d_tile_offsets, it.d_tile_max_lens, it.K, it.N, it.tile_height, it.tile_width = w.d_tile_offsets, w.d_tile_max_lens, K, N, 1024, 32
        it.d_out_exp, it.d_checkpoints, it.segments = out.p, w.d_checkpoints, segs
    m.clear()
    m.call("ci_decode_tiled_ilp2_batch", items, len(shapes), None)
    # one tensor has whole streams of 512 rows: the whole batch runs on the whole-stream kernel
    assert m.launches() == ["decode_tiled32_persist_kernel<false>"], m.launches()
    for out, ref in zip(outs, refs):
        assert np.array_equal(out.get(), ref)


@in_child
def test_decode_batch_on_sixteen_wavefronts():
    """Several tensors with checkpoints in one launch of decode_tiled32_seg_kernel: every workgroup has to find its
    tensor in the batch (the CUs are divided among the tensors by their sizes)."""
    import ctypes as C

    from oracle import rans_oracle as ro
    from tests.hostmodel.model import DecodeItem

    for cus in (3, 8):
        m = Model(cus=cus)
        shapes = [(2048, 64, 2), (1024, 256, 4), (1500, 40, 2), (1024, 96, 8), (3072, 32, 2)]
        items = (DecodeItem * len(shapes))()
        keep, outs, refs = [], [], []
        for i, (K, N, segs) in enumerate(shapes):
            bits = weight_bits(K, N, 40 + i)
            enc, man = cases.compress(bits, 1024)
            w, kp = m.weight(enc, None, K, N, segments=segs)
            out = m.empty((K, N), np.uint8)
            keep.append((w, kp))
            outs.append(out)
            refs.append(ro.split_bf16(bits)[0])
            it = items[i]
            it.d_stream, it.stream_len, it.d_states, it.d_tables, it.d_slot_map = w.d_stream, w.stream_len, w.d_states, w.d_tables, w.d_slot_map
            it.d_tile_offsets, it.d_tile_max_lens, it.K, it.N, it.tile_height, it.tile_width = w.d_tile_offsets, w.d_tile_max_lens, K, N, 1024, 32
            it.d_out_exp, it.d_checkpoints, it.segments = out.p, w.d_checkpoints, segs
        m.clear()
        m.call("ci_decode_tiled_ilp2_batch", items, len(shapes), None)
        assert m.launches() == ["decode_tiled32_seg_kernel<false>"], m.launches()
        for out, ref in zip(outs, refs):
            assert np.array_equal(out.get(), ref)


@in_child
def test_decode_batch_with_an_empty_tensor_and_a_stream_at_an_odd_address():
    """A batch in which two tensors are empty (skipped) and one has its stream at an address that is no multiple of
    16: that one goes through the one-thread-per-stream kernel, which reads the stream a byte at a time, the rest
    through the batched launch."""
    import ctypes as C

    from oracle import rans_oracle as ro
    from tests.hostmodel.model import DecodeItem

    m = Model(cus=4)
    shapes = [(2048, 64, 2), (0, 64, 1), (1024, 96, 1), (1024, 0, 1)]
    items = (DecodeItem * len(shapes))()
    keep, outs, refs = [], [], []
    for i, (K, N, segs) in enumerate(shapes):
        it = items[i]
        it.K, it.N, it.tile_height, it.tile_width, it.segments = K, N, 1024, 32, segs
        if K == 0 or N == 0:
            continue  # (no pointer of an empty tensor is looked at)
        bits = weight_bits(K, N, 50 + i)
        enc, man = cases.compress(bits, 1024)
        w, kp = m.weight(enc, None, K, N, segments=segs)
        if i == 2:
            room = m.empty(enc.stream.size + 16, np.uint8)
            C.memmove(room.ptr + 8, enc.stream.ctypes.data, enc.stream.size)
            m.lib.sim_mark_written(C.c_void_p(room.ptr + 8), C.c_size_t(enc.stream.size))  # (the bytes around it stay unwritten)
            w.d_stream = room.ptr + 8
            keep.append(room)
        out = m.empty((K, N), np.uint8)
        keep.append((w, kp))
        outs.append(out)
        refs.append(ro.split_bf16(bits)[0])
        it.d_stream, it.stream_len, it.d_states, it.d_tables, it.d_slot_map = w.d_stream, w.stream_len, w.d_states, w.d_tables, w.d_slot_map
        it.d_tile_offsets, it.d_tile_max_lens = w.d_tile_offsets, w.d_tile_max_lens
        it.d_out_exp, it.d_checkpoints = out.p, w.d_checkpoints
    m.clear()
    m.call("ci_decode_tiled_ilp2_batch", items, len(shapes), None)
    assert m.launches() == ["(decode_tiled_generic_kernel<false, 2>)", "decode_tiled32_seg_kernel<false>"], m.launches()
    for out, ref in zip(outs, refs):
        assert np.array_equal(out.get(), ref)


# ---- fused linear -----------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("K,N,M,th,segs,prep,kernel", [
    (2048, 128, 1, 1024, 1, False, "fused_linear32_kernel<1>"),
    (2048, 128, 40, 1024, 1, False, "fused_linear32_kernel<2>"),
    (2048, 128, 3, 1024, 2, False, "fused_linear32_seg_kernel<1, true>"),
    (2048, 128, 3, 1024, 2, True, "fused_linear32_seg_kernel<1, false>"),    # M <= 4: sums handed over without a barrier
    (2048, 128, 9, 1024, 4, True, "fused_linear32_seg_kernel<1, false>"),
    (2048, 128, 64, 1024, 2, True, "fused_linear32_seg_kernel<2, false>"),
    (4096, 64, 2, 1024, 8, True, "fused_linear32_seg_kernel<1, false>"),     # 64 items per column tile: several rounds per job
    (2048, 320, 9, 256, 2, True, "fused_linear32_seg_kernel<1, false>"),     # ten jobs on four CUs: sums through the window areas, job after job
    (2048, 320, 40, 256, 2, True, "fused_linear32_seg_kernel<2, false>"),
    (2048, 320, 3, 256, 2, True, "fused_linear32_seg_kernel<1, false>"),     # ... and handed over without a barrier, job after job
    (1024, 320, 4, 256, 1, False, "fused_linear32_seg_kernel<1, true>"),     # low tiles, several column tiles per job
    (2048 + 100, 100, 5, 1024, 2, False, "fused_linear32_seg_kernel<1, true>"),  # ragged: guarded path inside the kernel
    (3072, 96, 7, 2048, 1, False, "fused_linear32_kernel<1>"),
    (2048, 95, 2, 1024, 2, True, "fused_linear32_seg_kernel<1, true>"),      # one column short of whole tiles
    (1024, 31, 40, 1024, 1, False, "fused_linear32_kernel<2>"),
    (2048, 128, 100, 1024, 2, True, "fused_linear32_kernel<2>"),             # above 64 rows the checkpoints are not used
])
@in_child
def test_fused_linear(K, N, M, th, segs, prep, kernel):
    cases.linear(Model(cus=4), weight_bits(K, N, 1), x_bits(M, K, 2), th, segs, slot_table=prep, window_rows=prep,
                 expect_kernel=kernel)


@pytest.mark.parametrize("M,kernel", [(2, "fused_linear32_resident_kernel<1>"), (40, "fused_linear32_resident_kernel<2>")])
@in_child
def test_fused_linear_resident_kernel(M, kernel):
    # segments of 512 rows: too long for the sixteen-wavefront kernel's windows, so every (tile, segment) is an item
    # of the twelve-wavefront resident kernel, whole bodies' windows transposed
    cases.linear(Model(cus=4), weight_bits(4096, 64, 1), x_bits(M, 4096, 2), 2048, 2, expect_kernel=kernel)


@pytest.mark.parametrize("M,kernel", [(65, "fused_linear32_wide_kernel<4>"), (128, "fused_linear32_wide_kernel<4>"),
                                      (129, "fused_linear32_wide_kernel<8>"), (300, "fused_linear32_wide_kernel<8>")])
@in_child
def test_fused_linear_above_64_rows_in_one_pass(M, kernel):
    """fused_linear32_wide_kernel: bit-identical to the 64-rows-a-pass kernel, which the twin check implies (the
    plain-weight twin always runs the 64-row kernel) and which is asserted directly as well."""
    import ctypes as C

    m = Model(cus=4)
    K, N, th = 2048, 96, 1024
    bits, xb = weight_bits(K, N, 1), x_bits(M, K, 2)
    cases.linear(m, bits, xb, th, wide=True, expect_kernel=kernel)
    cases.linear(m, bits, xb, th, wide=False, expect_kernel="fused_linear32_kernel<2>")
    # ragged weight: every tile of the last row and column takes the guarded path of the wide kernel
    cases.linear(m, weight_bits(K + 40, N - 6, 3), x_bits(M, K + 40, 2), th, wide=True, expect_kernel=kernel)


@in_child
def test_fused_linear_bias_row_stride_and_the_entry_point_without_allocation():
    m = Model(cus=4)
    K, N, th = 2048, 128, 1024
    bits, bias = weight_bits(K, N, 1), x_bits(1, N, 9)[0]
    for M, segs in ((1, 2), (33, 1), (5, 4)):
        cases.linear(m, bits, x_bits(M, K, 2), th, segs, bias=bias, x_pad=24, window_rows=True)
        cases.linear(m, bits, x_bits(M, K, 2), th, segs, bias=bias, noalloc=True, window_rows=True)


@in_child
def test_fused_linear_without_room_for_the_fragment_copy():
    """A workspace that holds the partial sums and nothing more (or no workspace where the plan has none): the
    kernels read x in place, the rows past the last one masked -- x ends at the inaccessible page."""
    m = Model(cus=4)
    bits = weight_bits(2048, 128, 1)
    for M, segs, prep, kernel in ((40, 2, True, "fused_linear32_seg_kernel<2, false>"), (64, 2, True, "fused_linear32_seg_kernel<2, false>"),
                                  (33, 4, False, "fused_linear32_seg_kernel<2, true>"), (20, 2, True, "fused_linear32_seg_kernel<1, false>"),
                                  (50, 1, False, "fused_linear32_kernel<2>"), (100, 1, False, "fused_linear32_kernel<2>")):
        launches = cases.linear(m, bits, x_bits(M, 2048, 2), 1024, segs, slot_table=prep, window_rows=prep, partials_only=True,
                                expect_kernel=kernel)
        assert "x_fragments_kernel" not in launches, launches
        m.free_all()


@pytest.mark.parametrize("kind", cases.KINDS)
@in_child
def test_fused_linear_on_unusual_planes(kind):
    rng = np.random.default_rng(12)
    bits = cases.weight_kind(rng, 2048, 96, kind)
    m = Model(cus=3)
    for M, segs, prep in ((1, 1, False), (2, 2, True), (40, 4, False), (100, 1, False)):
        cases.linear(m, bits, x_bits(M, 2048, 2), 1024, segs, slot_table=prep, window_rows=prep, wide=M > 64)


# ---- fused gather -----------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("K,N,n,th,segs,slot,kernel", [
    (4096, 128, 300, 1024, 1, False, "embed_gather32_kernel"),
    (4096, 128, 300, 1024, 8, False, "embed_gather32_kernel"),
    (4096, 128, 300, 1024, 8, True, "embed_gather32_seg_kernel"),
    (4096, 128, 300, 1024, 4, True, "embed_gather32_seg_kernel"),
    (5000, 100, 257, 1024, 8, True, "embed_gather32_seg_kernel"),   # ragged rows and columns, odd last column tile
    (3000, 96, 1, 512, 4, True, "embed_gather32_seg_kernel"),
    (4096, 95, 100, 1024, 8, True, "embed_gather32_seg_kernel"),    # one column short of whole tiles
    (2048, 63, 100, 1024, 1, False, "embed_gather32_kernel"),
    (4096, 63, 100, 1024, 8, True, "embed_gather32_seg_kernel"),    # ... of a whole pair of tiles
    (2048, 127, 64, 1024, 8, False, "embed_gather32_kernel"),
    (70000, 64, 2048, 1024, 8, True, "embed_gather32_seg_kernel"),
    (270000, 32, 500, 32, 1, False, "embed_sort_kernel<true>"),      # more buckets than counting slots: the sort
    (530000, 32, 500, 32, 1, False, "embed_sort_kernel<false>"),     # ... of ids that do not fit the packed key (2^19 rows and more)
    (2048, 32, 8192, 1024, 4, True, "embed_gather32_seg_kernel"),    # exactly one pass of ids: no second, empty pass
    (2048, 32, 8192 + 3, 1024, 1, False, "embed_gather32_kernel"),   # a second pass of three ids
    (300000, 32, 16384, 32, 1, False, "embed_sort_kernel"),          # two whole passes through the sort
])
@in_child
def test_fused_gather(K, N, n, th, segs, slot, kernel):
    rng = np.random.default_rng(4)
    ids = cases.zipf_ids(rng, K, n)
    if n > 8:
        ids[1], ids[5], ids[7] = -3, K, K + 12345678901  # outside the table: zero rows
        ids[2] = ids[3] = ids[4]                          # duplicates
    cases.gather(Model(cus=4), weight_bits(K, N, 3), ids, th, segs, slot, expect_kernel=kernel)


@pytest.mark.parametrize("kind", cases.KINDS)
@in_child
def test_fused_gather_on_unusual_planes(kind):
    rng = np.random.default_rng(13)
    bits = cases.weight_kind(rng, 6000, 96, kind)
    m = Model(cus=3)
    for segs, slot in ((1, False), (8, True), (4, True)):
        cases.gather(m, bits, rng.integers(0, 6000, 400), 1024, segs, slot)
        cases.gather(m, bits, np.full(70, 4095), 1024, segs, slot)  # one row asked for seventy times, the last of its tile


# ---- LM head ----------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("V,H,M,th,segs,prep,matrix,kernel", [
    (2048, 128, 1, 1024, 1, False, False, "trans32_kernel<1>"),
    (2048, 128, 3, 1024, 1, False, False, "trans32_kernel<kTrRows>"),
    (2048, 96, 6, 1024, 1, False, False, "trans32_kernel<kTrRows>"),
    (2048, 128, 1, 1024, 2, True, False, "trans32_seg_kernel<false>"),
    (2048, 128, 1, 1024, 4, True, False, "trans32_seg_kernel<false>"),
    (2048 + 300, 128, 1, 1024, 2, True, False, "trans32_seg_kernel<false>"),   # short last tile row: trans32_kernel takes it
    (2048, 128, 1, 1024, 2, True, True, "trans32_seg_kernel<true>"),
    (2048 + 300, 256, 1, 1024, 4, True, True, "trans32_seg_kernel<true>"),
    (2000, 100, 2, 512, 1, False, False, "trans32_kernel<kTrRows>"),
    (2048, 96, 1, 1024, 2, True, False, "trans32_seg_kernel<false>"),          # three column tiles
    (2048, 160, 1, 1024, 4, True, True, "trans32_seg_kernel<true>"),
    (2048 + 500, 64, 1, 1024, 4, True, False, "trans32_seg_kernel<false>"),    # a deep ragged tile row does not count in max_window_rows
    (500, 64, 1, 1024, 4, True, False, "trans32_kernel<1>"),                   # no whole tile row: nothing for the segment kernel
])
@in_child
def test_lm_head(V, H, M, th, segs, prep, matrix, kernel):
    cases.lm_head(Model(cus=4), weight_bits(V, H, 3), x_bits(M, H, 2), th, segs, slot_table=prep, window_rows=prep,
                  matrix_sums=matrix, expect_kernel=kernel, check_twin=not matrix)


@pytest.mark.parametrize("kind", cases.KINDS)
@in_child
def test_lm_head_on_unusual_planes(kind):
    rng = np.random.default_rng(14)
    bits = cases.weight_kind(rng, 2048, 64, kind)
    m = Model(cus=3)
    cases.lm_head(m, bits, x_bits(1, 64, 2), 1024)
    cases.lm_head(m, bits, x_bits(1, 64, 2), 1024, 2, window_rows=True)
    cases.lm_head(m, bits, x_bits(1, 64, 2), 1024, 4, window_rows=True, slot_table=True, matrix_sums=True, check_twin=False)


# ---- inputs at the edges of what a caller may pass ----------------------------------------------------------------------
@in_child
def test_empty_inputs_launch_nothing():
    """No rows of x, no ids, an empty shape: CI_OK and not one launch (a grid of zero workgroups is an error on the GPU)."""
    import ctypes as C

    m = Model(cus=4)
    K, N, th = 2048, 64, 1024
    enc, man = cases.compress(weight_bits(K, N, 1), th)
    w, keep = m.weight(enc, man, K, N, segments=2, slot_table=True, window_rows=True)
    buf = m.empty(4096, np.uint8)
    big = C.c_size_t(4096)
    m.clear()
    m.call("ci_fused_linear_tiled", C.byref(w), buf.p, 0, K, None, buf.p, N, buf.p, big, None)
    m.call("ci_fused_linear_tiled_noalloc", C.byref(w), buf.p, 0, K, None, buf.p, N, None)
    m.call("ci_fused_embedding_tiled", C.byref(w), buf.p, 0, buf.p, N, buf.p, big, None)
    m.call("ci_fused_linear_transposed_tiled", C.byref(w), buf.p, 0, N, None, buf.p, K, buf.p, big, None)
    m.call("ci_splitk_reduce", buf.p, 0, 3, 0, N, None, buf.p, N, None)
    m.call("ci_splitk_reduce", buf.p, 0, 3, 5, 0, None, buf.p, 0, None)
    body = (keep["stream"].p, C.c_uint64(enc.stream.size), keep["states"].p, keep["tables"].p, keep["slot_map"].p,
            keep["offs"].p, keep["lens"].p)
    m.call("ci_decode_tiled_ilp2", *body, 0, N, th, 32, buf.p, None, None, None)
    m.call("ci_decode_tiled_ilp2", *body, K, 0, th, 32, buf.p, None, None, None)
    m.call("ci_fused_linear_ilp2", buf.p, 3, K, 0, K, *body, keep["man"].p, th, 32, None, buf.p, 0, buf.p, big, None)
    m.call("ci_build_checkpoints_ilp2", *body, 0, N, th, 32, 2, buf.p, big, None)
    m.call("ci_build_checkpoints_ilp2", *body, K, 0, th, 32, 2, buf.p, big, None)
    m.call("ci_fused_embedding_ilp2", buf.p, 3, *body, keep["man"].p, K, 0, th, 32, buf.p, 0, buf.p, big, None)
    m.call("ci_fused_linear_transposed_ilp2", buf.p, 1, N, 0, N, *body, keep["man"].p, th, 32, None, buf.p, 0, buf.p, big, None)
    m.call("ci_fused_linear_transposed_ilp2", buf.p, 0, N, K, N, *body, keep["man"].p, th, 32, None, buf.p, K, buf.p, big, None)
    assert m.launches() == [], m.launches()


@in_child
def test_a_stream_that_is_not_16_byte_aligned():
    """The whole-tile and sixteen-wavefront kernels load the stream 16 bytes at a time; a stream at another address
    (a view into a larger buffer) goes through the kernels that read it byte by byte, with the same results."""
    import ctypes as C

    from oracle import rans_oracle as ro
    from tests.hostmodel.model import bf16_bits_to_f32

    m = Model(cus=4)
    K, N, th = 2048, 96, 1024
    bits = weight_bits(K, N, 1)
    enc, man = cases.compress(bits, th)
    w, keep = m.weight(enc, man, K, N)
    for shift in (8, 4, 1):
        room = m.empty(enc.stream.size + 16, np.uint8)
        C.memmove(room.ptr + shift, enc.stream.ctypes.data, enc.stream.size)
        m.lib.sim_mark_written(C.c_void_p(room.ptr + shift), C.c_size_t(enc.stream.size))  # (the bytes around it stay unwritten)
        w.d_stream = room.ptr + shift
        out = m.empty((K, N), np.uint8)
        xb = x_bits(3, K, 2)
        x, y = m.dev(xb), m.empty((3, N), np.uint16)
        nb = m.lib.ci_fused_linear_workspace_bytes(3, K, N, th, 32, 0)
        ws = m.empty(max(nb, 16), np.uint8)
        ids = np.array([0, 7, 2047, 1024, -1], np.int64)
        g = m.empty((ids.size, N), np.uint16)
        nbe = m.lib.ci_fused_embedding_workspace_bytes(ids.size, K, th)
        wse = m.empty(max(nbe, 16), np.uint8)
        xh = x_bits(1, N, 2)
        z = m.empty((1, K), np.uint16)
        nbt = m.lib.ci_fused_linear_transposed_workspace_bytes(1, N, K, 32)
        wst = m.empty(max(nbt, 16), np.uint8)
        m.clear()
        m.call("ci_decode_tiled", C.byref(w), out.p, None, None)
        m.call("ci_fused_linear_tiled", C.byref(w), x.p, 3, K, None, y.p, N, ws.p, C.c_size_t(nb), None)
        m.call("ci_fused_embedding_tiled", C.byref(w), m.dev(ids).p, ids.size, g.p, N, wse.p, C.c_size_t(nbe), None)
        m.call("ci_fused_linear_transposed_tiled", C.byref(w), m.dev(xh).p, 1, N, None, z.p, K, wst.p, C.c_size_t(nbt), None)
        assert not any(k.startswith(("decode_tiled32", "fused_linear32", "embed_gather32", "trans32")) for k in m.launches()), m.launches()
        assert np.array_equal(out.get(), ro.split_bf16(bits)[0])
        assert np.allclose(bf16_bits_to_f32(y.get()), ro.linear_f32(xb, bits), atol=1e-2, rtol=1e-2)
        want = np.zeros((ids.size, N), np.uint16)
        want[:4] = bits[ids[:4]]
        assert np.array_equal(g.get(), want)
        assert np.allclose(bf16_bits_to_f32(z.get()), ro.linear_f32(xh, np.ascontiguousarray(bits.T)), atol=1e-2, rtol=1e-2)


# ---- split-K reduction ------------------------------------------------------------------------------------------------
@in_child
def test_splitk_reduction_in_index_order():
    """ci_splitk_reduce: out = bf16(sum over the planes in index order (+ bias)), fp32 and bf16 partials, through both
    kernels (one output a thread; four a thread from 65,536 outputs on) and through every stage of their unrolled
    loops (16 / 4 / 1 planes at a time, 8 / 1): bit for bit the sequential fp32 sum."""
    import ctypes as C

    from tests.hostmodel.model import bf16_bits_to_f32, f32_to_bf16_bits

    m = Model(cus=4)
    rng = np.random.default_rng(8)
    for P, M, N in ((1, 3, 40), (3, 5, 33), (4, 2, 64), (7, 1, 96), (16, 2, 50), (21, 3, 36), (37, 1, 128),
                    (9, 64, 1024), (16, 128, 512), (23, 33, 2048)):
        part = (rng.standard_normal((P, M, N), dtype=np.float32) * 3).astype(np.float32)
        bias = f32_to_bf16_bits(rng.standard_normal(N, dtype=np.float32))
        want = np.zeros((M, N), np.float32)
        for p in range(P):
            want = (want + part[p]).astype(np.float32)
        for with_bias in (False, True):
            # (the sum is rounded to bf16 and the bias added in bf16, as torch.sum(...) then `+= bias` do in the reference)
            w = (bf16_bits_to_f32(f32_to_bf16_bits(want)) + bf16_bits_to_f32(bias)[None, :]).astype(np.float32) if with_bias else want
            out = m.empty((M, N + 8), np.uint16)
            b = m.dev(bias)
            m.clear()
            m.call("ci_splitk_reduce", m.dev(part).p, 0, P, M, N, b.p if with_bias else None, out.p, N + 8, None)
            kernel = "splitk_reduce4_kernel" if M * N >= 65536 and N % 4 == 0 else "splitk_reduce_kernel"
            assert m.launches() == [kernel], (m.launches(), P, M, N)
            assert np.array_equal(out.get()[:, :N], f32_to_bf16_bits(w)), (P, M, N, with_bias)
        # the reference's workspace: bf16 partials [S, M, N] (comp_inference/linear_triton.py:303-314)
        pb = f32_to_bf16_bits(part)
        want = np.zeros((M, N), np.float32)
        for p in range(P):
            want = (want + bf16_bits_to_f32(pb[p])).astype(np.float32)
        out = m.empty((M, N), np.uint16)
        m.call("ci_splitk_reduce", m.dev(pb).p, 1, P, M, N, None, out.p, N, None)
        assert np.array_equal(out.get(), f32_to_bf16_bits(want)), (P, M, N, "bf16 partials")
        m.free_all()


# ---- which path ran -------------------------------------------------------------------------------------------------
@in_child
def test_the_hand_scheduled_loops_are_what_these_tests_run():
    """Every kernel has a guarded path in C++ that gives the same results as its hand-scheduled loop, so a test that
    compares results cannot tell which of the two ran -- and the loop is what the GPU will run.  The model counts the
    assembly instructions it interprets: on whole tiles of ordinary weights, prepared as the runtime prepares them,
    all decode steps must have gone through the statements (0.95 to 1.1 times the loops' instructions per step: prologues and tails add a few per cent) (decode 20 instructions a step,
    fused linear 19.5, the eight-step block of the LM head 17, the gather's advance 18)."""
    m = Model(cus=4)
    K, N, th = 2048, 128, 1024
    wave_steps = (K // th) * (N // 32) * (th // 2)
    bits = weight_bits(K, N, 1)

    def share(per_step, run):
        run()  # (every case clears the model's records, the instruction count among them, before its call)
        got = m.asm_instructions() / (wave_steps * per_step)
        m.free_all()
        return got

    for segs, kernel in ((1, "decode_tiled32_persist_kernel<false>"), (2, "decode_tiled32_seg_kernel<false>"), (8, "decode_tiled32_seg_kernel<false>")):
        s = share(20, lambda: cases.decode(m, bits, th, segs, expect_kernel=kernel))
        assert 0.95 <= s <= 1.1, (kernel, segs, s)
    for M, segs, prep, kernel in ((1, 1, False, "fused_linear32_kernel<1>"), (40, 1, False, "fused_linear32_kernel<2>"),
                                  (1, 2, True, "fused_linear32_seg_kernel<1, false>"), (3, 4, False, "fused_linear32_seg_kernel<1, true>"),
                                  (64, 2, True, "fused_linear32_seg_kernel<2, false>"), (16, 8, True, "fused_linear32_seg_kernel<1, false>")):
        s = share(19.5, lambda: cases.linear(m, bits, x_bits(M, K, 2), th, segs, slot_table=prep, window_rows=prep,
                                             expect_kernel=kernel, check_twin=False))
        assert 0.95 <= s <= 1.15, (kernel, M, segs, s)
    for M, kernel in ((129, "fused_linear32_wide_kernel<8>"), (70, "fused_linear32_wide_kernel<4>")):
        s = share(17, lambda: cases.linear(m, bits, x_bits(M, K, 2), th, wide=True, expect_kernel=kernel, check_twin=False))
        assert 0.95 <= s <= 1.1, (kernel, s)
    s = share(19.5, lambda: cases.linear(m, weight_bits(4096, 64, 1), x_bits(2, 4096, 2), 2048, 2,
                                         expect_kernel="fused_linear32_resident_kernel<1>", check_twin=False))
    assert 0.95 <= s <= 1.15, ("resident", s)   # (4096 x 64 at tile height 2048: the same number of steps)
    for segs, prep, matrix, kernel in ((1, False, False, "trans32_kernel<1>"), (2, True, False, "trans32_seg_kernel<false>"),
                                       (4, True, True, "trans32_seg_kernel<true>")):
        s = share(17, lambda: cases.lm_head(m, bits, x_bits(1, N, 2), th, segs, slot_table=prep, window_rows=prep,
                                            matrix_sums=matrix, check_twin=False, expect_kernel=kernel))
        assert 0.95 <= s <= 1.1, (kernel, s)
    # the gather decodes every bucket it is asked about down to the deepest row asked for: all rows of the table here
    ids = np.arange(K, dtype=np.int64)
    for segs, slot, kernel in ((1, False, "embed_gather32_kernel"), (8, False, "embed_gather32_kernel"), (8, True, "embed_gather32_seg_kernel")):
        s = share(18, lambda: cases.gather(m, bits, ids, th, segs, slot, expect_kernel=kernel))
        assert s >= 0.95, (kernel, segs, s)


# ---- encoders and the other layouts --------------------------------------------------------------------------------------
@pytest.mark.parametrize("layout,th,tw", [("ilp2", 1024, 32), ("ilp2", 64, 16), ("one", 256, 32), ("one", 128, 64),
                                          ("dense", 512, 32)])
@in_child
def test_encoders(layout, th, tw):
    from oracle import rans_oracle as ro

    m = Model(cus=4)
    for K, N, seed in ((1500, 100, 1), (th, tw, 2), (2 * th + 1, 3 * tw + 5, 3)):
        cases.encode(m, ro.split_bf16(weight_bits(K, N, seed))[0], th, tw, layout)


@pytest.mark.parametrize("K,N,min_block", [(300, 8, 512), (512, 33, 512), (1500, 16, 512), (1024, 5, 256), (1, 1, 512)])
@in_child
def test_flat_layout_encoder_and_decoders(K, N, min_block):
    """a8, the legacy layout (512-row segments, bytes strided by the stream count, a checkpoint every 128 symbols): the
    library's encoder and packer against the oracle's, every output array compared, and both decoders on the result."""
    import ctypes as C

    from oracle import rans_oracle as ro

    m = Model(cus=4)
    exp = ro.split_bf16(weight_bits(K, N, 7))[0]
    f, c = ro.get_lut(exp)
    want = ro.encode_flat(exp, f, c, min_block)
    S, cap = C.c_uint32(0), C.c_uint32(0)
    m.call("ci_flat_geometry", K, N, min_block, C.byref(S), C.byref(cap))
    assert S.value == want.num_streams
    nb = m.lib.ci_encode_scratch_bytes(S.value, cap.value)
    sym, scratch = m.dev(exp), m.empty(nb, np.uint8)
    states, sizes, ck = m.empty(S.value, np.uint32), m.empty(S.value, np.uint32), m.empty(S.value * 128, np.uint64)
    f16, c16 = np.ascontiguousarray(f, np.uint16), np.ascontiguousarray(c, np.uint16)
    max_len = C.c_uint32(0)
    m.call("ci_encode_flat", sym.p, K, N, S.value, cap.value, f16.ctypes.data_as(C.c_void_p), c16.ctypes.data_as(C.c_void_p),
           scratch.p, C.c_size_t(nb), states.p, sizes.p, ck.p, C.byref(max_len), None)
    assert "max_len_kernel" in m.launches()
    stream = m.empty(max_len.value * S.value, np.uint8)
    m.call("ci_pack_flat", scratch.p, S.value, cap.value, sizes.p, max_len.value, stream.p, None)
    assert np.array_equal(states.get(), want.states) and np.array_equal(sizes.get(), want.sizes)
    assert np.array_equal(stream.get(), want.stream), "packed stream differs from the oracle's"
    assert np.array_equal(ck.get(), want.checkpoints), "checkpoints differ from the oracle's"
    tables, slot_map = m.dev(want.tables), m.dev(want.slot_map)
    out = m.empty((K, N), np.uint8)
    m.clear()
    m.call("ci_decode_flat_segmented", stream.p, C.c_uint64(stream.nbytes), states.p, sizes.p, S.value, tables.p, slot_map.p,
           K, N, out.p, None)
    assert any("decode_flat_kernel" in k for k in m.launches()), m.launches()
    assert np.array_equal(out.get(), exp), "segmented decode differs from the plane"
    # the extension's decoder: symbol i of stream g at g + i * streams
    flat = m.empty(K * N, np.uint8)
    m.call("ci_decode_flat_strided", stream.p, C.c_uint64(stream.nbytes), states.p, sizes.p, S.value, tables.p, slot_map.p,
           C.c_uint64(K * N), flat.p, None)
    assert np.array_equal(flat.get(), ro.decode_flat_strided(want.stream, want.states, want.sizes, want.tables, want.slot_map, K * N))


@pytest.mark.parametrize("layout,th,tw", [("one", 256, 32), ("one", 64, 16), ("one", 1024, 128), ("dense", 512, 32),
                                          ("ilp2", 128, 64), ("ilp2", 32, 16)])
@in_child
def test_operators_of_the_other_layouts(layout, th, tw):
    """a7 (one stream per column in tile bodies), the dense layout and other tile widths of the default layout: decode,
    fused linear, gather and LM head through the one-thread-per-stream kernels."""
    rng = np.random.default_rng(15)
    K, N = 2 * th + th // 2 + 3, 3 * tw + 7   # a last tile row of more than half a tile, less than a whole one
    ids = rng.integers(-2, K + 2, 37)
    ids[:4] = (K, K - 1, -1, K + 1)           # the first row past the table, the last row in it
    launches = cases.other_layout_ops(Model(cus=4), weight_bits(K, N, 5), x_bits(3, max(K, N), 2)[:, :K], ids, th, tw, layout)
    assert any("generic_kernel" in k for k in launches), launches


# ---- descriptors that promise too much ------------------------------------------------------------------------------------
@in_child
def test_an_understated_window_leaves_items_out_and_reads_nothing_out_of_bounds():
    """max_window_rows smaller than the truth selects the kernel instances without guarded path; an item whose window
    does not fit is then left out (fused linear) or gets zeros (LM head): wrong sums, as the header says, and no
    access outside the arrays or the window areas."""
    import ctypes as C

    m = Model(cus=4)
    rng = np.random.default_rng(3)
    K, N, th, segs = 2048, 64, 1024, 2
    bits = cases.weight_kind(rng, K, N, "wide")  # deep bodies: windows of more than 112 rows
    enc, man = cases.compress(bits, th)
    w, keep = m.weight(enc, man, K, N, segments=segs, slot_table=True, window_rows=True)
    assert w.max_window_rows > 112, w.max_window_rows
    w.max_window_rows = 7  # the lie
    x, y = m.dev(x_bits(1, K, 2)), m.empty((1, N), np.uint16)
    nb = m.lib.ci_fused_linear_workspace_bytes_segmented(1, K, N, th, 32, 0, segs)
    ws = m.empty(max(nb, 16), np.uint8)
    m.clear()
    m.call("ci_fused_linear_tiled", C.byref(w), x.p, 1, K, None, y.p, N, ws.p, C.c_size_t(nb), None)
    assert m.launches() == ["(fused_linear32_seg_kernel<1, false>)"], m.launches()
    # the LM head on the same arrays read as a [V = 2048, H = 64] table
    xh, z = m.dev(x_bits(1, N, 2)), m.empty((1, K), np.uint16)
    nbt = m.lib.ci_fused_linear_transposed_workspace_bytes(1, N, K, 32)
    wst = m.dev(np.full(nbt // 4, np.float32(np.nan)))  # what an earlier launch might have left in the workspace
    m.clear()
    m.call("ci_fused_linear_transposed_tiled", C.byref(w), xh.p, 1, N, None, z.p, K, wst.p, C.c_size_t(nbt), None)
    assert "trans32_seg_kernel<false>" in m.launches()
    from tests.hostmodel.model import bf16_bits_to_f32

    assert np.isfinite(bf16_bits_to_f32(z.get())).all(), "rows of a refused item surfaced as stale workspace contents"


@in_child
def test_tile_metadata_that_points_past_the_stream_is_not_followed():
    """Every kernel treats a tile body that would run past stream_len as empty instead of reading it."""
    import ctypes as C

    m = Model(cus=4)
    K, N, th = 2048, 96, 1024
    bits = weight_bits(K, N, 1)
    enc, man = cases.compress(bits, th)
    bad = enc.tile_offsets.copy()
    bad[-1] = enc.stream.size - 64      # the last body now ends beyond the stream
    bad[2] = 0xFFFFFF00                  # and one starts far outside it
    enc.tile_offsets = bad
    for segs, slot in ((1, False), (2, True)):
        w, keep = m.weight(enc, man, K, N, segments=segs, slot_table=slot)
        out, x, y = m.empty((K, N), np.uint8), m.dev(x_bits(2, K, 2)), m.empty((2, N), np.uint16)
        nb = m.lib.ci_fused_linear_workspace_bytes_segmented(2, K, N, th, 32, 0, segs)
        ws = m.empty(max(nb, 16), np.uint8)
        ids = m.dev(np.arange(0, K, 37, dtype=np.int64))
        n_ids = ids.shape[0]
        g = m.empty((n_ids, N), np.uint16)
        nbe = m.lib.ci_fused_embedding_workspace_bytes_segmented(n_ids, K, th, segs)
        wse = m.empty(nbe, np.uint8)
        z = m.empty((1, K), np.uint16)
        nbt = m.lib.ci_fused_linear_transposed_workspace_bytes(1, N, K, 32)
        wst = m.empty(nbt, np.uint8)
        m.clear()
        m.call("ci_decode_tiled", C.byref(w), out.p, None, None)
        m.call("ci_fused_linear_tiled", C.byref(w), x.p, 2, K, None, y.p, N, ws.p, C.c_size_t(nb), None)
        m.call("ci_fused_embedding_tiled", C.byref(w), ids.p, n_ids, g.p, N, wse.p, C.c_size_t(nbe), None)
        m.call("ci_fused_linear_transposed_tiled", C.byref(w), m.dev(x_bits(1, N, 2)).p, 1, N, None, z.p, K, wst.p, C.c_size_t(nbt), None)
        m.free_all()


@in_child
def test_the_bounded_wait_gives_up_and_says_so():
    """fused_linear32_seg_kernel for up to four rows of x: a wavefront waits for the one adding up the previous job.
    With the number of looks forced to zero (ci_debug_wait_limit) every such wait gives up without looking at its
    flag: the kernel still ends, the device status word says so, ci_device_status returns an error once and is clear
    after.  With the default limit the word stays clear."""
    import ctypes as C

    m = Model(cus=1)  # one workgroup takes every job in turn: waits between jobs
    m.lib.ci_debug_wait_limit.restype = C.c_uint32
    K, N, th, segs = 768, 200, 256, 2
    bits = weight_bits(K, N, 1)
    st = C.c_uint32(7)
    cases.linear(m, bits, x_bits(2, K, 2), th, segs)
    assert m.lib.ci_device_status(C.byref(st), None) == 0 and st.value == 0
    before = m.lib.ci_debug_wait_limit(0)
    assert before == 1 << 22
    try:
        try:
            cases.linear(m, bits, x_bits(2, K, 2), th, segs)  # the sums may or may not survive: not the point
        except AssertionError as e:
            assert "differs" in str(e) or "max error" in str(e), e
        assert m.violations() == []
        rc = m.lib.ci_device_status(C.byref(st), None)
        assert rc == 2 and st.value == 1 and b"bounded wait" in m.lib.ci_last_error(), (rc, st.value)
        assert m.lib.ci_device_status(C.byref(st), None) == 0 and st.value == 0
    finally:
        m.lib.ci_debug_wait_limit(before)


@in_child
def test_tile_bodies_without_a_byte():
    """A constant exponent plane in low tiles: no stream emits a byte, every tile body has depth 0, every window is
    empty.  The sixteen-wavefront kernels decode such items like any other (nothing to stage, no byte ever asked for)."""
    rng = np.random.default_rng(1)
    V, H, th = 384, 64, 128
    bits = cases.weight_kind(rng, V, H, "constant")
    enc, _ = cases.compress(bits, th)
    assert not enc.tile_max_lens.any() and enc.stream.size == 0
    m = Model(cus=2)
    cases.lm_head(m, bits, x_bits(1, H, 2), th, 2, window_rows=True, expect_kernel="trans32_seg_kernel<false>")
    cases.lm_head(m, bits, x_bits(1, H, 2), th, 2, window_rows=True, matrix_sums=True, check_twin=False,
                  expect_kernel="trans32_seg_kernel<true>")
    cases.linear(m, bits, x_bits(1, V, 2), th, 2, window_rows=True, slot_table=True, expect_kernel="fused_linear32_seg_kernel<1, false>")
    cases.decode(m, bits, th, 2, expect_kernel="decode_tiled32_seg_kernel<false>")
    cases.gather(m, bits, np.arange(0, V, 5), th, 2, slot_table=True, expect_kernel="embed_gather32_seg_kernel")


# ---- the reference's own parity sweep ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("th", [32, 64, 128, 256, 512, 1024])
@in_child
def test_reference_tile_sweep(th):
    """tests/test_mat_mul.py:108-264 of the reference: K = 3072 (a multiple of every height), tile heights 32..1024 x
    widths 16..128, fused result and decode-then-matmul against the product on the decompressed weight within
    allclose(1e-2, 1e-2).  Here with a quarter of the columns and 24 rows of x instead of 8192 (the CPU model's pace)."""
    from oracle import rans_oracle as ro

    m = Model(cus=8)
    K, N, M = 3072, 256, 24
    bits, xb = weight_bits(K, N, th), x_bits(M, K, 2)
    for tw in (16, 32, 64, 128):
        if tw == 32:
            cases.decode(m, bits, th, merge=True)
            cases.linear(m, bits, xb, th)
        else:
            cases.other_layout_ops(m, bits, xb, np.arange(0, K, 97), th, tw, "ilp2")
        m.free_all()
