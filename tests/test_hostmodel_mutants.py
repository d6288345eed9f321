"""Does the host model (tests/hostmodel) notice a mistake in the REAL kernels?  Each case builds the library with one
deliberate slip of a kind that is easy to make in this code -- a wait that covers one load too few, a prefetch that
does not wrap at the end of its tile, a lane-exchange control in the wrong direction, a row stored one position down,
a work-space size one group short -- runs the ordinary test case of that operator, and requires that
it fails, and by which means: the interpreter's load tracking, the exact extents of the arrays, the inaccessible page
behind an array, or the comparison with the oracle.  (The self-check file shows the same detectors on made-up kernels;
this one shows that the library's own code paths run through them.)

The last group takes barriers and release / acquire pairs out of the real kernels.  Such a kernel still computes the
right sums in the model, where the wavefronts run one after the other, and nothing of the plain build notices; the
build that checks the ordering between wavefronts (build.py, `order=True`) must."""
import numpy as np
import pytest

from tests.hostmodel import build, cases
from tests.hostmodel.model import Model, in_child, weight_bits, x_bits

MUTANTS = {
    # the pack of rows 0/1 waits for all but FIVE of the loads in flight; six lets the row-1 dword be used too early
    "wait_one_load_short": dict(
        edits=[("fast_tile.h", '"s_waitcnt vmcnt(5)\\n" CI_PACK("v72", "v74", C0, C1, "v108")',
                '"s_waitcnt vmcnt(6)\\n" CI_PACK("v72", "v74", C0, C1, "v108")')],
        rebuild=["linear.hip"], op="linear", expect="before the s_waitcnt"),
    # the loads of the block after the last wrap to block 0 so that they stay inside the tile
    "prefetch_runs_off_the_plane": dict(
        edits=[("fast_tile.h", """                                                uint32_t nblocks, uint32_t qdec = 1) {
    const uint32_t wrap_m = 0u - (nblocks - 1) * 256u, wrap_x = 0u - (nblocks - 1) * xstep;""",
                """                                                uint32_t nblocks, uint32_t qdec = 1) {
    const uint32_t wrap_m = 0x100u, wrap_x = 0u - (nblocks - 1) * xstep;""")],
        rebuild=["linear.hip"], op="linear", expect="outside every allocation"),
    # row_shl:4 / row_shr:4 pick the other four-lane group of a row: swapped, every sum takes the wrong partner
    "lane_exchange_direction": dict(
        edits=[("transposed.hip", "dpp_add<0x104>(t0), c1 = dpp_add<0x114>(t1)", "dpp_add<0x114>(t0), c1 = dpp_add<0x104>(t1)")],
        rebuild=["transposed.hip"], op="lm_head", expect="LM head"),
    # a gathered row goes to the position its id came from
    "row_stored_one_position_down": dict(
        edits=[("embedding.hip", "a.out[(size_t)p * a.out_stride + col] = (uint16_t)assemble_bf16(sym, man_cur[u]);",
                "a.out[(size_t)(p + 1) * a.out_stride + col] = (uint16_t)assemble_bf16(sym, man_cur[u]);", 2)],
        rebuild=["embedding.hip"], op="gather", expect=("memory fault", "gathered rows differ")),
    # --- in the kernels that have not run on a GPU yet ---
    # more than 64 rows in one pass: the last block loads its own operands again instead of the block after the tile's end
    "one_pass_kernel_prefetches_past_the_tile": dict(
        edits=[("linear.hip", "const uint32_t nb = blk + 1 < nblk ? blk + 1 : blk;  // (the last block re-reads its own: stays inside the tile)",
                "const uint32_t nb = blk + 1;")],
        rebuild=["linear.hip"], op="wide", expect=("memory fault", "outside every allocation")),
    # the gather on sixteen wavefronts stages windows as they lie: a lane's next byte is 64 bytes down, not 1
    "gather_window_pointer_step": dict(
        edits=[("embedding.hip", "sym = advance_asm(st, want + 1 - done, 64) >> 24;", "sym = advance_asm(st, want + 1 - done, 1) >> 24;")],
        rebuild=["embedding.hip"], op="gather16", expect=("gathered rows differ", "reads LDS address")),
    # the head's sums on the matrix pipe: the second block of a pair belongs to columns 8..15 / 24..31 of the one-hot operand
    "one_hot_operands_swapped": dict(
        edits=[("transposed.hip", "const u32x4 hot0 = mine && (n % 16) / 8 == 0 ? one : none, hot1 = mine && (n % 16) / 8 == 1 ? one : none;",
                "const u32x4 hot0 = mine && (n % 16) / 8 == 1 ? one : none, hot1 = mine && (n % 16) / 8 == 0 ? one : none;")],
        rebuild=["transposed.hip"], op="lm_head_matrix", expect="LM head"),
    # the fragment copy of x holds whole groups of 32 rows
    "fragment_copy_one_group_short": dict(
        edits=[("linear.hip", "    return M > 32 ? 2 * ceil_div(M, 64u) : 1u;", "    return M > 32 ? 2 * ceil_div(M, 64u) - 1 : 1u;")],
        rebuild=["linear.hip"], op="linear64", expect=("outside every allocation", "memory fault", "max error", "differs")),
}


# Synchronisation taken out: (edits, rebuild, case).  Right results, no violation in the plain build; reported by the
# build that checks the ordering between wavefronts.
ORDER_MUTANTS = {
    # the sums of a job go through the wavefronts' window areas, rows 32..63 of x after rows 0..31: a wavefront that is
    # ahead writes its second sums while a slower one still reads the first (with one group of rows the barrier orders
    # nothing that the one at the end of the job before has not ordered: a wavefront writes into its own window area)
    "sums_overwritten_while_still_read": dict(
        edits=[("linear.hip", "            __syncthreads();  // the window areas are free: every wavefront has left its loop\n", "")],
        rebuild=["linear.hip"], op="linear_two_jobs", plain_build_sees_it_too=True),  # (wrong sums in wavefront order as well)
    # few rows of x: the area of the sums is handed from job to job by a flag; stored without release semantics, the next
    # job's sums are not ordered after the additions that read the area
    "handover_flag_without_release": dict(
        edits=[("linear.hip", "__hip_atomic_store(&flags[1], jn + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);",
                "__hip_atomic_store(&flags[1], jn + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);")],
        rebuild=["linear.hip"], op="linear_small_m_two_jobs"),
    # more than 64 rows in one pass: the groups of rows share one area for their sums
    "one_pass_kernel_groups_share_the_area": dict(
        edits=[("linear.hip", "        if (g) __syncthreads();\n#pragma unroll\n        for (int v = 0; v < 16; ++v) red[(size_t)wave * frag + v * kWave + lane] = acc[g][v];",
                "#pragma unroll\n        for (int v = 0; v < 16; ++v) red[(size_t)wave * frag + v * kWave + lane] = acc[g][v];")],
        rebuild=["linear.hip"], op="wide_two_k_tiles"),
    # the gather on sixteen wavefronts decodes with the slot table the whole workgroup has copied into the LDS
    "slot_table_read_before_it_is_complete": dict(
        edits=[("embedding.hip", """        if (h1) emb_request(a, r1, pr1, lane, raw);
    }
    __syncthreads();
    while (h0) {""", """        if (h1) emb_request(a, r1, pr1, lane, raw);
    }
    while (h0) {""")],
        rebuild=["embedding.hip"], op="gather16"),
    # the LM head on sixteen wavefronts gives an item it must refuse (a descriptor that understates the largest window)
    # zeros; without them the reduction adds up whatever an earlier launch left in those rows of the workspace -- in
    # the model the fill pattern of a fresh array, a tiny number as fp32: every tolerance passes
    "refused_item_leaves_its_rows_of_the_workspace_unwritten": dict(
        edits=[("transposed.hip", "            for (uint32_t i = c; i < min(seglen, a.V - v0); i += 32) a.partial[(size_t)tn * a.V + v0 + i] = 0.f;\n",
                "            ;\n")],
        rebuild=["transposed.hip"], op="lm_head_understated_window", says="nothing has written"),
}


def _run(op: str, lib_path: str):
    m = Model(cus=2, lib_path=lib_path)
    if op == "linear":
        cases.linear(m, weight_bits(2048, 64, 1), x_bits(3, 2048, 2), 1024, 2, slot_table=True, window_rows=True)
    elif op in ("linear_two_jobs", "linear_small_m_two_jobs"):  # four column tiles on two CUs: two jobs a workgroup
        cases.linear(m, weight_bits(2048, 128, 1), x_bits(40 if op == "linear_two_jobs" else 3, 2048, 2), 256, 2,
                     slot_table=True, window_rows=True, expect_kernel="fused_linear32_seg_kernel")
    elif op == "linear64":
        cases.linear(m, weight_bits(1024, 64, 1), x_bits(40, 1024, 2), 1024)
    elif op == "lm_head":
        cases.lm_head(m, weight_bits(2048, 64, 1), x_bits(1, 64, 2), 1024, check_twin=False)
    elif op == "wide":
        cases.linear(m, weight_bits(1024, 64, 1), x_bits(129, 1024, 2), 1024, wide=True, expect_kernel="fused_linear32_wide_kernel")
    elif op == "wide_two_k_tiles":  # two wavefronts add their sums for one column tile
        cases.linear(m, weight_bits(2048, 64, 1), x_bits(129, 2048, 2), 1024, wide=True, expect_kernel="fused_linear32_wide_kernel")
    elif op == "lm_head_understated_window":
        import ctypes as C

        rng = np.random.default_rng(3)
        V, H, th, segs = 2048, 64, 1024, 2
        enc, man = cases.compress(cases.weight_kind(rng, V, H, "wide"), th)  # deep bodies: windows of more than 112 rows
        w, keep = m.weight(enc, man, V, H, segments=segs, slot_table=True, window_rows=True)
        assert w.max_window_rows > 112
        w.max_window_rows = 7  # the lie: every item is refused
        x, z = m.dev(x_bits(1, H, 2)), m.empty((1, V), np.uint16)
        nb = m.lib.ci_fused_linear_transposed_workspace_bytes(1, H, V, 32)
        ws = m.empty(nb // 4, np.float32)  # (a fresh array: nothing written)
        m.call("ci_fused_linear_transposed_tiled", C.byref(w), x.p, 1, H, None, z.p, V, ws.p, C.c_size_t(nb), None)
        assert "trans32_seg_kernel<false>" in m.launches()
    elif op == "gather16":
        ids = np.arange(0, 2048, 3, dtype=np.int64)
        cases.gather(m, weight_bits(2048, 64, 1), ids, 1024, 8, slot_table=True, expect_kernel="embed_gather32_seg_kernel")
    elif op == "lm_head_matrix":
        cases.lm_head(m, weight_bits(2048, 64, 1), x_bits(1, 64, 2), 1024, 2, slot_table=True, window_rows=True,
                      matrix_sums=True, check_twin=False, expect_kernel="trans32_seg_kernel<true>")
    elif op == "gather":
        ids = np.array([0, 5, 2047, 2048, 1024, 7, -1, 2047], np.int64)
        cases.gather(m, weight_bits(2048, 64, 1), ids, 1024)  # (two column tiles: the hand-scheduled path)


@pytest.fixture(scope="module")
def libraries():
    # the compilations of all mutants side by side
    from concurrent.futures import ThreadPoolExecutor

    build.build()
    with ThreadPoolExecutor(len(MUTANTS)) as pool:
        futures = {tag: pool.submit(build.build_mutant, tag, mu["edits"], mu["rebuild"]) for tag, mu in MUTANTS.items()}
        return {tag: f.result() for tag, f in futures.items()}


def test_the_cases_pass_on_the_intact_library():
    for op in sorted({mu["op"] for mu in MUTANTS.values()}):
        in_child(_run)(op, build.build())


@pytest.mark.parametrize("tag", sorted(MUTANTS))
def test_a_mistake_in_the_kernels_is_noticed(libraries, tag, capfd):
    mu = MUTANTS[tag]
    with pytest.raises(AssertionError) as caught:
        in_child(_run)(mu["op"], libraries[tag])
    said = str(caught.value) + capfd.readouterr().err
    expect = mu["expect"] if isinstance(mu["expect"], tuple) else (mu["expect"],)
    assert any(e in said for e in expect), said[-1500:]


@pytest.fixture(scope="module")
def order_libraries():
    from concurrent.futures import ThreadPoolExecutor

    build.build()
    build.build(order=True)
    with ThreadPoolExecutor(2 * len(ORDER_MUTANTS)) as pool:
        futures = {(tag, order): pool.submit(build.build_mutant, tag, mu["edits"], mu["rebuild"], order)
                   for tag, mu in ORDER_MUTANTS.items() for order in (False, True)}
        return {key: f.result() for key, f in futures.items()}


def test_the_cases_pass_on_the_intact_library_that_checks_ordering():
    for op in sorted({mu["op"] for mu in ORDER_MUTANTS.values()}):
        in_child(_run)(op, build.build(order=True))


@pytest.mark.parametrize("tag", sorted(ORDER_MUTANTS))
def test_synchronisation_taken_out_is_noticed_by_the_ordering_check(order_libraries, tag):
    mu = ORDER_MUTANTS[tag]
    if not mu.get("plain_build_sees_it_too"):
        in_child(_run)(mu["op"], order_libraries[tag, False])  # right results, nothing reported: the wavefronts run one after the other
    with pytest.raises(AssertionError) as caught:
        in_child(_run)(mu["op"], order_libraries[tag, True])
    assert "ordering:" in str(caught.value) and mu.get("says", "") in str(caught.value), str(caught.value)[-1500:]
