"""Host-side logic that needs no GPU, and the C ABI: the shared library loads and exports every
function that include/comp_inference_hip.h declares (no compute calls here)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from helpers import bf16_bits, bits_to_bf16, make_weight_kn, make_x

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "comp_inference_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ci_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from comp_inference_amd import _lib

    lib = _lib.lib()
    names = _declared_functions()
    assert len(names) >= 15
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in the header but not exported"


def test_every_exported_entry_point_is_declared():
    import subprocess

    from comp_inference_amd import _lib

    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True).stdout
    exported = sorted(set(re.findall(r"\bT (ci_[a-z0-9_]+)", out)))
    assert exported == _declared_functions()


def test_host_only_entry_points_run_without_gpu():
    from comp_inference_amd import _lib

    lib = _lib.lib()
    assert lib.ci_abi_version() >= 1
    t = _lib.Tiling()
    assert lib.ci_tiling_init(ctypes.byref(t), 4096, 14336, 1024, 32, 1) == 0
    assert (t.num_tiles_k, t.num_tiles_n, t.num_tiles, t.num_streams) == (4, 448, 1792, 114688)
    assert t.capacity == int(512 * 1.25) + 64  # src/cuda/rans_host.cuh:470-471
    assert lib.ci_tiling_init(ctypes.byref(t), 128256, 4096, 1024, 32, 1) == 0
    assert (t.num_tiles_k, t.num_tiles) == (126, 16128)
    # tile height not a multiple of 16 is refused with the reference's message (rans_host.cuh:441-445)
    assert lib.ci_tiling_init(ctypes.byref(t), 4096, 4096, 24, 32, 1) != 0
    assert b"tile height" in lib.ci_last_error()
    assert lib.ci_tiling_init(ctypes.byref(t), 0, 4096, 1024, 32, 1) != 0
    # decoder tables built on the host equal the oracle's
    from oracle import rans_oracle as ro

    f, c = ro.get_lut(np.arange(256, dtype=np.uint8).repeat(3))
    tables, slot_map = np.zeros(256, np.uint32), np.zeros(4096, np.uint8)
    vp = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    assert lib.ci_build_tables(vp(f), vp(c), vp(tables), vp(slot_map)) == 0
    to, so = ro.build_tables(f, c)
    assert np.array_equal(tables, to) and np.array_equal(slot_map, so)
    bad = c.copy()
    bad[255] = 4095
    f2 = f.copy()
    f2[255] = 9
    assert lib.ci_build_tables(vp(f2), vp(bad), vp(tables), vp(slot_map)) != 0


def test_ops_refuse_cpu_tensors():
    """There is no CPU path: ops given host tensors raise instead of computing."""
    from comp_inference_amd import ccore, fused_rans_linear_triton, rans_decomp_triton_tiled

    z8, z32 = torch.zeros(64, dtype=torch.uint8), torch.zeros(64, dtype=torch.int32)
    with pytest.raises(RuntimeError):
        rans_decomp_triton_tiled(z8, z32, z32, z8, (1024, 32), z32, z32)
    with pytest.raises(RuntimeError):
        fused_rans_linear_triton(torch.zeros(1, 1024, dtype=torch.bfloat16), z8, z32, z32, z8, (1024, 32), z32, z32,
                                 1024, 32, z8)
    with pytest.raises(RuntimeError, match="GPU"):
        ccore.decompress(z8, z32, z32, 64, z32, z8, z8)
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError):
            ccore.RansManager().compress_tiled(torch.zeros(1024, 32, dtype=torch.uint8), z32, z32, 1024, 32)


def test_reference_numerics_restatement_is_within_the_reference_tolerance(oracle):
    """The reference rounds each product to bf16 and stores bf16 split partials; its own test
    accepts atol=rtol=1e-2 against an fp32 matmul (tests/test_mat_mul.py:220)."""
    K, N, M = 2048, 64, 4
    w = make_weight_kn(N, K, 3)
    x = make_x(M, K, 4)
    ref = bits_to_bf16(oracle.linear_reference_numerics(bf16_bits(x), bf16_bits(w), None, 1024, 8)).float()
    f32 = torch.from_numpy(oracle.linear_f32(bf16_bits(x), bf16_bits(w)))
    f64 = (x.double() @ w.double()).float()
    assert torch.allclose(f32, f64, atol=1e-4, rtol=1e-4)
    assert torch.allclose(ref, f64, atol=1e-2, rtol=1e-2)
    bias = make_x(1, N, 5).view(N)
    refb = bits_to_bf16(oracle.linear_reference_numerics(bf16_bits(x), bf16_bits(w), bf16_bits(bias), 1024, 8))
    assert torch.equal(refb, (ref.to(torch.bfloat16) + bias))


def test_embedding_oracle_equals_table_lookup(oracle):
    K, N, th, tw = 1300, 64, 512, 32
    table = make_weight_kn(N, K, 7)  # [K, N]
    enc, man = oracle.compress_bf16(bf16_bits(table), th, tw)
    ids = np.array([0, 1, 255, 256, 511, 512, 1023, 1024, 1299, 1300, -1, 7, 7], np.int64)
    got = oracle.embedding_gather(ids, enc, man, K, N)
    want = np.zeros((ids.size, N), np.uint16)
    ok = (ids >= 0) & (ids < K)
    want[ok] = bf16_bits(table)[ids[ok]]
    assert np.array_equal(got, want)


def test_every_linear_plan_that_writes_partial_sums_has_a_workspace():
    """The one-thread-per-stream kernel (one-stream-per-column layout, tile widths other than 32, unaligned
    streams) writes fp32 partial sums for the reduction kernel even when there is a single one per output
    -- the one-stream-per-column layout with K <= tile_height.  The size query must cover that case, and
    the entry point must refuse a missing workspace before anything is launched (checked here with
    made-up, never dereferenced device addresses: no GPU is touched)."""
    from comp_inference_amd import _lib

    lib = _lib.lib()
    M, N = 3, 96
    for K, th, dense, planes in ((1024, 1024, 1, 1), (700, 1024, 1, 1), (4096, 1024, 1, 4), (1024, 1024, 0, 2),
                                 (4096, 1024, 0, 8)):
        need = lib.ci_fused_linear_workspace_bytes(M, K, N, th, 32, dense)
        assert need >= planes * M * N * 4, (K, th, dense, need)
    fake = ctypes.c_void_p(0x1000)
    for K in (1024, 700):
        rc = lib.ci_fused_linear_dense(fake, M, K, N, K, fake, ctypes.c_uint64(64), fake, fake, fake, fake, fake, fake,
                                       1024, 32, None, fake, N, None, ctypes.c_size_t(0), None)
        assert rc == 3 and b"workspace" in lib.ci_last_error(), K      # CI_ERR_CAPACITY
        rc = lib.ci_fused_linear_dense(fake, M, K, N, K, fake, ctypes.c_uint64(64), fake, fake, fake, fake, fake, fake,
                                       1024, 32, None, fake, N, fake, ctypes.c_size_t(M * N * 4 - 1), None)
        assert rc == 3, K


def test_operand_sizes_are_checked_before_a_kernel_sees_them():
    """The kernels index states, offsets and tables by tile and stream without a bound of their own; the
    Python operators refuse arrays of the wrong length (ValueError, like the reference's decoder,
    comp_inference/rans_triton.py:141-144)."""
    from comp_inference_amd._lib import check_tiled_operands as chk

    z = lambda n: torch.zeros(n, dtype=torch.int32)  # noqa: E731
    chk(1300, 80, 1024, 32, z(2 * 3 * 64), z(256), z(4096), z(6), z(6), False)           # 2 x 3 tiles
    chk(1300, 80, 1024, 32, z(2 * 3 * 32), z(256), z(4096), z(192), z(192), True)         # one stream per column
    for bad in (lambda: chk(1300, 80, 1024, 32, z(383), z(256), z(4096), z(6), z(6), False),
                lambda: chk(1300, 80, 1024, 32, z(384), z(256), z(4096), z(5), z(6), False),
                lambda: chk(1300, 80, 1024, 32, z(384), z(256), z(4096), z(6), z(7), False),
                lambda: chk(1300, 80, 1024, 32, z(384), z(255), z(4096), z(6), z(6), False),
                lambda: chk(1300, 80, 1024, 32, z(384), z(256), z(4095), z(6), z(6), False),
                lambda: chk(1300, 80, 1024, 32, z(192), z(256), z(4096), z(6), z(6), True)):
        with pytest.raises(ValueError):
            bad()


def test_entry_points_refuse_bad_arguments_before_any_launch():
    """Argument checks come before the first HIP call, so they can be exercised without a GPU: made-up,
    never dereferenced device addresses; every call must come back with CI_ERR_ARG (1) or
    CI_ERR_CAPACITY (3) and a message."""
    from comp_inference_amd import _lib

    lib = _lib.lib()
    P = ctypes.c_void_p
    fake, null = P(0x1000), P(0)
    u64, sz = ctypes.c_uint64, ctypes.c_size_t
    K, N, M = 14336, 96, 2

    def lin(ws, ws_bytes, th=1024, x_stride=K, states=fake, segs=None, ck=null):
        head = (fake, M, K, N, x_stride, fake, u64(64), states, fake, fake, fake, fake, fake, th, 32)
        tail = (None, fake, N, ws, sz(ws_bytes), None)
        if segs is None:
            return lib.ci_fused_linear_ilp2(*head, *tail)
        return lib.ci_fused_linear_ilp2_segmented(*head, ck, segs, *tail)

    need = lib.ci_fused_linear_workspace_bytes(M, K, N, 1024, 32, 0)
    assert need >= 2 * M * N * 4
    assert lin(null, 0) == 3 and b"workspace" in lib.ci_last_error()          # 14 k-tiles: two partial sums
    assert lin(fake, 2 * M * N * 4 - 1) == 3
    assert lin(fake, need, th=1023) == 1                                       # odd tile height
    assert lin(fake, need, x_stride=K - 8) == 1                                # row stride shorter than the row
    assert lin(fake, need, states=null) == 1
    assert lin(fake, need, segs=4, ck=null) == 1                               # segments without checkpoints
    assert lin(fake, need, segs=3, ck=fake) == 1                               # 512 rows do not split in 3 x 16 n
    assert lin(fake, need, segs=4, ck=P(0x1004)) == 1                          # checkpoints not 8-byte aligned

    V, H = 5000, 256
    tneed = lib.ci_fused_linear_transposed_workspace_bytes(M, H, V, 32)
    assert tneed == (H // 32) * M * V * 4

    def trans(ws, ws_bytes, x_stride=H):
        return lib.ci_fused_linear_transposed_ilp2(fake, M, H, V, x_stride, fake, u64(64), fake, fake, fake, fake, fake, fake,
                                                   1024, 32, None, fake, V, ws, sz(ws_bytes), None)

    assert trans(null, 0) == 3 and trans(fake, tneed - 1) == 3 and trans(fake, tneed, x_stride=H - 1) == 1

    def emb(ws, ws_bytes, out_stride=H, segs=None, ck=null, th=1024):
        head = (fake, 7, fake, u64(64), fake, fake, fake, fake, fake, fake, V, H, th, 32)
        tail = (fake, out_stride, ws, sz(ws_bytes), None)
        if segs is None:
            return lib.ci_fused_embedding_ilp2(*head, *tail)
        return lib.ci_fused_embedding_ilp2_segmented(*head, ck, segs, *tail)

    eneed = lib.ci_fused_embedding_workspace_bytes(7, V, 1024)
    assert eneed > 7 * 8
    assert emb(null, 0) == 3 and emb(fake, eneed - 1) == 3
    assert emb(fake, eneed, out_stride=H - 1) == 1
    assert emb(fake, eneed, segs=8, ck=null) == 1 and emb(fake, eneed, segs=3, ck=fake) == 1
    assert emb(fake, eneed, th=1023) == 1

    def dec(out, th=1024, segs=None, ck=null, states=fake):
        head = (fake, u64(64), states, fake, fake, fake, fake, 2048, 64, th, 32)
        if segs is None:
            return lib.ci_decode_tiled_ilp2(*head, out, None, None, None)
        return lib.ci_decode_tiled_ilp2_segmented(*head, ck, segs, out, None, None, None)

    assert dec(null) == 1 and dec(fake, th=1023) == 1 and dec(fake, states=null) == 1
    assert dec(fake, segs=4, ck=null) == 1 and dec(fake, segs=3, ck=fake) == 1
    assert lib.ci_build_checkpoints_ilp2(fake, u64(64), fake, fake, fake, fake, fake, 2048, 64, 1024, 32, 4, fake,
                                         sz(lib.ci_checkpoint_bytes(2048, 64, 1024, 32, 4) - 1), None) == 3
    assert lib.ci_build_checkpoints_ilp2(fake, u64(64), fake, fake, fake, fake, fake, 2048, 64, 1024, 32, 3, fake,
                                         sz(1 << 20), None) == 1                # 512 rows do not split in 3
    assert lib.ci_splitk_reduce(null, 0, 4, M, N, None, fake, N, None) == 1
    assert lib.ci_splitk_reduce(fake, 0, 4, M, N, None, fake, N - 1, None) == 1
    assert lib.ci_last_error() != b""


def test_suggested_segments_for_the_shapes_they_were_chosen_on():
    """ci_suggest_segments: the fewest segments per stream that make an item 256 rows or less and the items enough to
    fill a chip of 256 CUs x 16 wavefronts; 1 where the tile shape allows none.  The figures the measurements were
    taken with (Llama-3-8B projections at tile 1024 x 32)."""
    from comp_inference_amd import _lib

    lib = _lib.lib()
    lib.ci_suggest_segments.restype = ctypes.c_uint32
    for (K, N, th, tw), want in {(4096, 14336, 1024, 32): 2, (4096, 28672, 1024, 32): 2, (14336, 4096, 1024, 32): 2,
                                 (128256, 4096, 1024, 32): 2, (4096, 6144, 1024, 32): 4, (4096, 4096, 1024, 32): 8,
                                 (4096, 1024, 1024, 32): 8, (4096, 64, 2048, 32): 16, (4096, 1024, 256, 32): 2,
                                 (512, 64, 64, 32): 1, (4096, 4096, 1000, 32): 1, (4096, 4096, 1024, 64): 1,
                                 (4096, 4096, 0, 32): 1}.items():
        assert lib.ci_suggest_segments(K, N, th, tw) == want, (K, N, th, tw)


def test_every_required_pointer_and_size_is_checked():
    """One argument at a time made NULL (or zero, or misaligned) in an otherwise acceptable call of every
    bare-pointer entry point of the default format: CI_ERR_ARG each time, before any HIP call.  The acceptable
    call itself gets past the checks (and fails at the first HIP call here, where there is no GPU)."""
    from comp_inference_amd import _lib

    lib = _lib.lib()
    P, u64, sz = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_size_t
    fake, null, odd = P(0x10000), P(0), P(0x10002)
    big = sz(1 << 30)

    def sweep(name, args, required, zero_is_bad=(), misaligned=()):
        fn = getattr(lib, name)
        assert fn(*args) != 1, (name, lib.ci_last_error())  # past the argument checks
        for i in required:
            bad = list(args)
            bad[i] = null
            assert fn(*bad) == 1, (name, "argument", i, "NULL was accepted")
            assert lib.ci_last_error() != b""
        for i in zero_is_bad:
            bad = list(args)
            bad[i] = 0
            assert fn(*bad) == 1, (name, "argument", i, "0 was accepted")
        for i in misaligned:
            bad = list(args)
            bad[i] = odd
            assert fn(*bad) == 1, (name, "argument", i, "a misaligned pointer was accepted")

    K, N, M, th = 2048, 96, 3, 1024
    body = (fake, u64(4096), fake, fake, fake, fake, fake)  # stream, its length, states, tables, slot_map, two per-tile arrays
    # d_x M K N x_stride | body | man th tw bias out out_stride ws ws_bytes stream
    lin = (fake, M, K, N, K) + body + (fake, th, 32, None, fake, N, fake, big, None)
    sweep("ci_fused_linear_ilp2", lin, required=(0, 5, 7, 8, 9, 10, 11, 12, 16), zero_is_bad=(2, 13, 14), misaligned=(9,))
    sweep("ci_fused_linear_dense", lin, required=(0, 5, 7, 8, 9, 10, 11, 12, 16), zero_is_bad=(2, 13, 14), misaligned=(9,))
    sweep("ci_fused_linear_one", lin, required=(0, 5, 7, 8, 9, 10, 11, 12, 16), zero_is_bad=(2, 13, 14), misaligned=(9,))
    seg = lin[:15] + (fake, 2) + lin[15:]
    sweep("ci_fused_linear_ilp2_segmented", seg, required=(0, 5, 7, 8, 9, 10, 11, 12, 15, 18), zero_is_bad=(2, 13, 14), misaligned=(9, 15))
    # d_x M H V x_stride | body | man th tw bias out out_stride ws ws_bytes stream
    head = (fake, 1, 96, 2048, 96) + body + (fake, th, 32, None, fake, 2048, fake, big, None)
    sweep("ci_fused_linear_transposed_ilp2", head, required=(0, 5, 7, 8, 9, 10, 11, 12, 16), zero_is_bad=(2, 13, 14), misaligned=(9,))
    sweep("ci_fused_linear_transposed_dense", head, required=(0, 5, 7, 8, 9, 10, 11, 12, 16), zero_is_bad=(2, 13, 14), misaligned=(9,))
    # ids n_ids | body | man K N th tw out out_stride ws ws_bytes stream
    emb = (fake, 7) + body + (fake, K, N, th, 32, fake, N, fake, big, None)
    sweep("ci_fused_embedding_ilp2", emb, required=(0, 2, 4, 5, 6, 7, 8, 9, 14), zero_is_bad=(12, 13), misaligned=(6,))
    embs = emb[:14] + (fake, 8) + emb[14:]
    sweep("ci_fused_embedding_ilp2_segmented", embs, required=(0, 2, 4, 5, 6, 7, 8, 9, 14, 16), zero_is_bad=(12, 13), misaligned=(6, 14))
    # body | K N th tw out_exp man out_bf16 stream
    dec = body + (K, N, th, 32, fake, None, None, None)
    sweep("ci_decode_tiled_ilp2", dec, required=(0, 2, 3, 4, 5, 6, 11), zero_is_bad=(9, 10), misaligned=(4,))
    sweep("ci_decode_tiled_one", dec, required=(0, 2, 3, 4, 5, 6, 11), zero_is_bad=(9, 10), misaligned=(4,))
    decs = body + (K, N, th, 32, fake, 2, fake, None, None, None)
    sweep("ci_decode_tiled_ilp2_segmented", decs, required=(0, 2, 3, 4, 5, 6, 11, 13), zero_is_bad=(9, 10), misaligned=(4, 11))
    merged = body + (K, N, th, 32, None, fake, fake, None)  # the bf16 output needs the sign|mantissa plane
    sweep("ci_decode_tiled_ilp2", merged, required=(12, 13))
    # body | K N th tw segments ckpt bytes stream
    ck = body + (K, N, th, 32, 4, fake, big, None)
    sweep("ci_build_checkpoints_ilp2", ck, required=(0, 2, 3, 4, 5, 6, 12), zero_is_bad=(9, 10), misaligned=(4, 12))
    # tables slot_map out bytes stream
    sweep("ci_build_slot_table", (fake, fake, fake, sz(32768), None), required=(0, 1, 2), misaligned=(1, 2))


def test_shared_workspace_grows_and_is_reused():
    """RansWorkspace (comp_inference/pytorch_runtime.py:386-394): one buffer for all layers, twice the first request,
    handed out again while it is large enough and on the same device, replaced when a request outgrows it."""
    from comp_inference_amd.pytorch_runtime import RansWorkspace

    RansWorkspace._buffer = None
    a = RansWorkspace.get_workspace(4, 96, 8, "cpu")
    assert a.shape == (8, 4, 96) and a.dtype == torch.bfloat16 and RansWorkspace._buffer.numel() == 2 * 8 * 4 * 96
    first = RansWorkspace._buffer.data_ptr()
    b = RansWorkspace.get_workspace(8, 96, 8, "cpu")      # exactly what is there
    c = RansWorkspace.get_workspace(1, 32, 2, torch.device("cpu"))
    assert b.data_ptr() == c.data_ptr() == first and c.shape == (2, 1, 32)
    d = RansWorkspace.get_workspace(8, 96, 8 + 1, "cpu")  # one plane more than the buffer holds
    assert RansWorkspace._buffer.numel() == 2 * 9 * 8 * 96 and d.shape == (9, 8, 96)
    RansWorkspace._buffer = None


def test_size_queries_answer_zero_for_a_tile_shape_that_cannot_be():
    """A size query has no error code: a tile height or width of zero (and, for checkpoints, fewer than two
    segments) gives 0, not a division by zero; a usable shape gives a size."""
    from comp_inference_amd import _lib

    lib = _lib.lib()
    for name in ("ci_fused_linear_workspace_bytes", "ci_fused_linear_workspace_bytes_segmented", "ci_checkpoint_bytes",
                 "ci_fused_embedding_workspace_bytes", "ci_fused_embedding_workspace_bytes_segmented",
                 "ci_fused_linear_transposed_workspace_bytes"):
        getattr(lib, name).restype = ctypes.c_size_t
    K, N = 4096, 96
    for th, tw, ok in ((1024, 32, True), (0, 32, False), (1024, 0, False), (0, 0, False)):
        assert (lib.ci_fused_linear_workspace_bytes(3, K, N, th, tw, 0) != 0) == ok, (th, tw)
        assert (lib.ci_fused_linear_workspace_bytes_segmented(3, K, N, th, tw, 0, 2) != 0) == ok, (th, tw)
        assert (lib.ci_checkpoint_bytes(K, N, th, tw, 2) != 0) == ok, (th, tw)
    assert lib.ci_checkpoint_bytes(K, N, 1024, 32, 1) == 0 and lib.ci_checkpoint_bytes(K, N, 1024, 32, 0) == 0
    assert lib.ci_checkpoint_bytes(K, N, 1024, 32, 4) == 4 * 3 * 3 * 64 * 8  # tiles x (segments - 1) x 64 streams x 8 bytes
    assert lib.ci_fused_embedding_workspace_bytes(7, K, 0) == 0 and lib.ci_fused_embedding_workspace_bytes(7, K, 1024) != 0
    assert lib.ci_fused_linear_transposed_workspace_bytes(1, N, K, 0) == 0
    assert lib.ci_fused_linear_transposed_workspace_bytes(1, N, K, 32) != 0


def test_segment_counts_a_tile_height_does_not_allow_are_refused():
    """Checkpoints can cut half a tile into any number of equal runs (the builder and the gather take every divisor);
    the decode and the fused linear read whole 16-row blocks, so they take the counts whose runs are multiples of 16
    rows.  Everything else is CI_ERR_ARG before any HIP call; what is accepted gets past the checks."""
    from comp_inference_amd import _lib

    lib = _lib.lib()
    P, u64, sz = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_size_t
    fake, big = P(0x10000), sz(1 << 30)
    K, N = 4096, 96
    body = (fake, u64(4096), fake, fake, fake, fake, fake)

    def builder(th, segs):
        return lib.ci_build_checkpoints_ilp2(*body, K, N, th, 32, segs, fake, big, None)

    def gather(th, segs):
        return lib.ci_fused_embedding_ilp2_segmented(fake, 7, *body, fake, K, N, th, 32, fake, segs, fake, N, fake, big, None)

    def decode(th, segs):
        return lib.ci_decode_tiled_ilp2_segmented(*body, K, N, th, 32, fake, segs, fake, None, None, None)

    def linear(th, segs):
        return lib.ci_fused_linear_ilp2_segmented(fake, 3, K, N, K, *body, fake, th, 32, fake, segs, None, fake, N, fake, big, None)

    any_divisor = {(1024, 2): True, (1024, 64): True, (1024, 512): True, (1024, 3): False, (1024, 1024): False,
                   (1000, 4): True, (1000, 125): True, (1000, 8): False, (1023, 2): False, (96, 16): True, (96, 32): False}
    blocks_of_16 = {(1024, 2): True, (1024, 32): True, (1024, 64): False, (1024, 3): False, (1000, 4): False, (1000, 2): False,
                    (96, 3): True, (96, 2): False, (992, 31): True, (1023, 2): False, (2048, 64): True, (2048, 128): False}
    for fn, table in ((builder, any_divisor), (gather, any_divisor), (decode, blocks_of_16), (linear, blocks_of_16)):
        for (th, segs), accepted in table.items():
            rc = fn(th, segs)
            assert (rc != 1) == accepted, (fn.__name__, th, segs, rc, lib.ci_last_error())
    lib.ci_fused_embedding_workspace_bytes_segmented.restype = ctypes.c_size_t
    for (th, segs), accepted in any_divisor.items():
        assert (lib.ci_fused_embedding_workspace_bytes_segmented(7, K, th, segs) != 0) == accepted, (th, segs)
    assert lib.ci_fused_embedding_workspace_bytes_segmented(7, K, 1, 1) == 0
    assert lib.ci_fused_embedding_workspace_bytes_segmented(7, K, 2, 1) != 0


def test_public_header_is_plain_c(tmp_path):
    """The boundary is a C ABI: the header compiles as C99 on its own and a C program links against the
    library's host-only entry points."""
    import shutil
    import subprocess

    from comp_inference_amd import _lib

    if shutil.which("gcc") is None:
        pytest.skip("no C compiler")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = tmp_path / "use.c"
    src.write_text('#include "comp_inference_hip.h"\n'
                   "int main(void) {\n"
                   "    ci_tiling t;\n"
                   "    if (ci_tiling_init(&t, 4096, 14336, 1024, 32, 1) != 0 || t.num_tiles != 1792) return 1;\n"
                   "    if (ci_fused_linear_workspace_bytes(1, 14336, 4096, 1024, 32, 0) == 0) return 2;\n"
                   "    return ci_abi_version() >= 1 ? 0 : 3;\n"
                   "}\n")
    exe = tmp_path / "use"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(root, "include"),
                    str(src), "-o", str(exe), _lib.LIB_PATH, "-Wl,-rpath," + os.path.dirname(_lib.LIB_PATH),
                    "-Wl,-rpath,/opt/rocm/lib"], check=True)
    assert subprocess.run([str(exe)]).returncode == 0


def test_a_descriptor_with_a_short_array_is_refused_on_the_host():
    """ci_tiled_weight carries the length of every array; the check runs on the host alone, so every kind of short
    or missing array is tried here with made-up addresses, and the entry points that take a descriptor refuse it
    with CI_ERR_ARG (1) before any device call."""
    from comp_inference_amd import _lib

    lib = _lib.lib()
    K, N, th, tw = 4096, 96, 1024, 32
    tiles = (K // th) * (N // tw)

    def desc(**over):
        w = _lib.TiledWeight()
        w.K, w.N, w.tile_height, w.tile_width = K, N, th, tw
        w.d_stream, w.stream_len = 0x10000, 1 << 20
        w.d_states, w.n_states = 0x20000, tiles * 64
        w.d_tables, w.d_slot_map = 0x30000, 0x40000
        w.d_tile_offsets, w.d_tile_max_lens, w.n_tiles = 0x50000, 0x60000, tiles
        w.d_man_tiled, w.man_len = 0x70000, tiles * th * tw
        w.d_checkpoints, w.checkpoint_bytes, w.segments = None, 0, 1
        w.d_slot_table, w.slot_table_bytes, w.max_window_rows = None, 0, 0
        for k, v in over.items():
            setattr(w, k, v)
        return w

    def rc(**over):
        return lib.ci_tiled_weight_check(ctypes.byref(desc(**over)))

    assert rc() == 0
    assert rc(n_states=tiles * 64 - 1) == 1 and b"states" in lib.ci_last_error()
    assert rc(n_tiles=tiles - 1) == 1 and b"tile metadata" in lib.ci_last_error()
    assert rc(man_len=tiles * th * tw - 1) == 1 and b"mantissa" in lib.ci_last_error()
    assert rc(d_man_tiled=None, man_len=0) == 0            # exponent plane only
    assert rc(d_man_tiled=None) == 1
    assert rc(d_states=None) == 1 and rc(d_tile_offsets=None) == 1 and rc(d_stream=None) == 1
    assert rc(d_slot_map=0x40002) == 1                     # not 4-byte aligned
    assert rc(tile_height=1023) == 1 and rc(K=0) == 1
    for field in ("N", "tile_height", "tile_width"):
        assert rc(**{field: 0}) == 1, field
    for field in ("d_tables", "d_slot_map", "d_tile_max_lens"):
        assert rc(**{field: None}) == 1, field
    assert rc(d_slot_table=0x90008, slot_table_bytes=32768) == 1   # not 16-byte aligned
    ck = lib.ci_checkpoint_bytes(K, N, th, tw, 4)
    assert ck == tiles * 3 * 64 * 8
    assert rc(segments=4, d_checkpoints=0x80000, checkpoint_bytes=ck) == 0
    assert rc(segments=4, d_checkpoints=0x80000, checkpoint_bytes=ck - 8) == 1 and b"checkpoints" in lib.ci_last_error()
    assert rc(segments=4, d_checkpoints=None, checkpoint_bytes=ck) == 1
    assert rc(segments=4, d_checkpoints=0x80004, checkpoint_bytes=ck) == 1
    assert rc(d_slot_table=0x90000, slot_table_bytes=32768) == 0 and rc(d_slot_table=0x90000, slot_table_bytes=4096) == 1
    assert lib.ci_tiled_weight_check(None) == 1

    # every entry point that takes a descriptor checks it first
    fake = ctypes.c_void_p(0x1000)
    short = ctypes.byref(desc(n_states=5))
    sz = ctypes.c_size_t
    assert lib.ci_fused_linear_tiled(short, fake, 1, K, None, fake, N, fake, sz(1 << 20), None) == 1
    assert lib.ci_fused_linear_tiled_noalloc(short, fake, 1, K, None, fake, N, None) == 1
    assert lib.ci_fused_embedding_tiled(short, fake, 3, fake, N, fake, sz(1 << 20), None) == 1
    assert lib.ci_fused_linear_transposed_tiled(short, fake, 1, N, None, fake, K, fake, sz(1 << 20), None) == 1
    assert lib.ci_decode_tiled(short, fake, None, None) == 1
    assert lib.ci_max_window_rows(short, fake, None) == 1
    # operators that need the sign|mantissa plane refuse a weight without one
    bare = ctypes.byref(desc(d_man_tiled=None, man_len=0))
    assert lib.ci_fused_linear_tiled(bare, fake, 1, K, None, fake, N, fake, sz(1 << 20), None) == 1
    assert lib.ci_fused_embedding_tiled(bare, fake, 3, fake, N, fake, sz(1 << 20), None) == 1
    assert lib.ci_fused_linear_transposed_tiled(bare, fake, 1, N, None, fake, K, fake, sz(1 << 20), None) == 1
    assert lib.ci_decode_tiled(bare, None, fake, None) == 1


def test_one_stream_layout_host_checks():
    """The first tiled format (one stream per column and tile in tile bodies): operand lengths in Python, tiling
    and pointer checks of the entry points, all before any HIP call."""
    from comp_inference_amd import _lib
    from comp_inference_amd._lib import check_tiled_operands as chk

    z = lambda n: torch.zeros(n, dtype=torch.int32)  # noqa: E731
    chk(1300, 80, 1024, 32, z(2 * 3 * 32), z(256), z(4096), z(6), z(6), False, True)      # 2 x 3 tiles, 32 streams each
    for bad in (lambda: chk(1300, 80, 1024, 32, z(2 * 3 * 64), z(256), z(4096), z(6), z(6), False, True),
                lambda: chk(1300, 80, 1024, 32, z(192), z(256), z(4096), z(192), z(192), False, True),
                lambda: chk(1300, 80, 1024, 32, z(192), z(256), z(4095), z(6), z(6), False, True)):
        with pytest.raises(ValueError):
            bad()

    lib = _lib.lib()
    P = ctypes.c_void_p
    fake, null = P(0x1000), P(0)
    u64, sz = ctypes.c_uint64, ctypes.c_size_t
    two, one = _lib.Tiling(), _lib.Tiling()
    assert lib.ci_tiling_init(ctypes.byref(two), 2048, 64, 1024, 32, 1) == 0
    assert lib.ci_tiling_init(ctypes.byref(one), 2048, 64, 1024, 32, 0) == 0
    assert (one.streams_per_tile, one.num_streams, two.num_streams) == (32, 128, 256)
    total = u64(0)
    f = np.full(256, 16, np.uint16)
    c = (np.arange(256) * 16).astype(np.uint16)
    fp, cp = f.ctypes.data_as(P), c.ctypes.data_as(P)
    # a tiling made for the other layout is refused by both encoders and both packers
    assert lib.ci_encode_tiled_one(fake, ctypes.byref(two), fp, cp, fake, sz(1 << 30), fake, fake, fake, fake,
                                   ctypes.byref(total), None) == 1 and b"one stream" in lib.ci_last_error()
    assert lib.ci_encode_tiled_ilp2(fake, ctypes.byref(one), fp, cp, fake, sz(1 << 30), fake, fake, fake, fake,
                                    ctypes.byref(total), None) == 1 and b"two streams" in lib.ci_last_error()
    assert lib.ci_pack_tiled_one(fake, ctypes.byref(two), fake, fake, fake, fake, u64(64), None) == 1
    assert lib.ci_pack_tiled_ilp2(fake, ctypes.byref(one), fake, fake, fake, fake, u64(64), None) == 1
    assert lib.ci_pack_tiled_one(fake, ctypes.byref(one), fake, fake, fake, null, u64(64), None) == 1    # no stream buffer
    assert lib.ci_pack_tiled_one(fake, ctypes.byref(one), fake, fake, fake, null, u64(0), None) == 0     # nothing to pack
    # scratch too small: refused before the encode kernel (CI_ERR_CAPACITY)
    assert lib.ci_encode_tiled_one(fake, ctypes.byref(one), fp, cp, fake, sz(16), fake, fake, fake, fake,
                                   ctypes.byref(total), None) == 3

    def dec(out, states=fake, th=1024, man=None, out16=None):
        return lib.ci_decode_tiled_one(fake, u64(64), states, fake, fake, fake, fake, 2048, 64, th, 32, out, man, out16, None)

    assert dec(null) == 1 and dec(fake, states=null) == 1 and dec(fake, th=0) == 1
    assert dec(null, man=fake, out16=null) == 1                                  # merge asked without bf16 output
    assert lib.ci_decode_tiled_one(fake, u64(64), fake, fake, fake, fake, fake, 0, 64, 1024, 32, null, None, None, None) == 0

    M, K, N = 2, 2048, 64
    need = lib.ci_fused_linear_workspace_bytes(M, K, N, 1024, 32, 1)
    assert need >= 2 * M * N * 4                                                  # one partial per tile row

    def lin(ws, ws_bytes, x_stride=K, states=fake):
        return lib.ci_fused_linear_one(fake, M, K, N, x_stride, fake, u64(64), states, fake, fake, fake, fake, fake, 1024, 32,
                                       None, fake, N, ws, sz(ws_bytes), None)

    assert lin(null, 0) == 3 and lin(fake, need - 1) == 3 and lin(fake, need, x_stride=K - 1) == 1
    assert lin(fake, need, states=null) == 1
    assert lib.ci_fused_embedding_one(fake, 5, fake, u64(64), fake, fake, fake, fake, fake, fake, 2048, 64, 1024, 32, fake,
                                      63, None) == 1                              # row stride shorter than the row
    assert lib.ci_fused_embedding_one(fake, 5, fake, u64(64), null, fake, fake, fake, fake, fake, 2048, 64, 1024, 32, fake,
                                      64, None) == 1
    tneed = lib.ci_fused_linear_transposed_workspace_bytes(M, 64, 2048, 32)
    assert lib.ci_fused_linear_transposed_one(fake, M, 64, 2048, 64, fake, u64(64), fake, fake, fake, fake, fake, fake, 1024,
                                              32, None, fake, 2048, fake, sz(tneed - 1), None) == 3
    assert lib.ci_fused_linear_transposed_one(fake, M, 64, 2048, 63, fake, u64(64), fake, fake, fake, fake, fake, fake, 1024,
                                              32, None, fake, 2048, fake, sz(tneed), None) == 1


def test_wide_rows_switch_and_fragment_sizes():
    """ci_fused_linear_wide_rows returns the previous setting; the workspace of more than 64 rows holds the fragment
    copy of x padded to whole passes (4 groups of 32 rows up to 128 rows, 8 above), whichever kernel then runs."""
    from comp_inference_amd import _lib

    lib = _lib.lib()
    assert lib.ci_fused_linear_wide_rows(1) == 0 and lib.ci_fused_linear_wide_rows(0) == 1
    assert lib.ci_fused_linear_wide_rows(0) == 0
    assert lib.ci_fused_linear_transposed_matrix_sums(1) == 0 and lib.ci_fused_linear_transposed_matrix_sums(0) == 1
    assert lib.ci_fused_linear_transposed_matrix_sums(0) == 0
    K, N = 4096, 256
    size = lambda M: lib.ci_fused_linear_workspace_bytes(M, K, N, 1024, 32, 0)  # noqa: E731
    # (sized for the one-thread-per-stream plan too: 8 partial sums per output, then the fragment copy)
    want = lambda M, groups: 8 * M * N * 4 + groups * 32 * K * 2  # noqa: E731
    assert size(64) == want(64, 2)
    assert size(65) == want(65, 4) and size(128) == want(128, 4)
    assert size(129) == want(129, 8) and size(256) == want(256, 8)
    assert size(257) == want(257, 16)
