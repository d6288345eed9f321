"""The host model checks itself: kernels that make one mistake on purpose (tests/hostmodel/selftest.hip) must be
reported, and what the model computes for the lane exchanges and the matrix instruction is compared with values
written out by hand from the instruction set's definition.  (That the model agrees with the GPU where it matters
is shown by the library's kernels that have run on the GPU giving the oracle's results in the model too: the other
test_hostmodel_* files.)"""
import ctypes as C

import numpy as np
import pytest

from tests.hostmodel.model import Model, bf16_bits_to_f32, f32_to_bf16_bits, in_child


def _u32(m, n):
    return m.empty(n, np.uint32)


@in_child
def test_an_assembly_load_is_checked_against_the_exact_extent_of_the_arrays():
    m = Model()
    src = m.dev(np.arange(100, 150, dtype=np.uint32))
    dst = _u32(m, 64)
    m.lib.simtest_global_load(src.p, 50, dst.p, 0)
    assert m.violations() == []
    assert np.array_equal(dst.get(), 2 * (100 + np.arange(64) % 50))
    m.lib.simtest_global_load(src.p, 50, dst.p, 1)  # lane 7: its own 28 bytes + the 200 of the array: checked before the access
    v = m.violations()
    assert len(v) == 1 and "lane 7" in v[0] and "outside every allocation" in v[0] and "offset 228" in v[0], v


@in_child
def test_a_register_used_before_its_waitcnt_is_reported():
    m = Model()
    src, dst = m.dev(np.arange(64, dtype=np.uint32)), _u32(m, 64)
    m.lib.simtest_global_load(src.p, 64, dst.p, 2)
    assert any("before the s_waitcnt" in s for s in m.violations()), m.violations()


@in_child
def test_a_scalar_operand_that_differs_between_lanes_is_reported():
    m = Model()
    src, dst = m.dev(np.arange(64, dtype=np.uint32)), _u32(m, 64)
    m.lib.simtest_global_load(src.p, 32, dst.p, 3)
    assert any("scalar register but differs between lanes" in s for s in m.violations()), m.violations()


@in_child
def test_lds_reads_of_the_interpreter_are_bounded_by_the_launch():
    m = Model()
    dst = _u32(m, 64)
    m.lib.simtest_lds_read(dst.p, 256, 0)
    assert m.violations() == [] and np.array_equal(dst.get(), (np.arange(64) * 3) & 0xFF)
    m.lib.simtest_lds_read(dst.p, 256, 1)
    assert any("lane 5 reads LDS address 0x100" in s for s in m.violations()), m.violations()
    m.clear()
    m.lib.simtest_lds_read(dst.p, 256, 2)
    assert any("still in flight" in s for s in m.violations()), m.violations()


@in_child
def test_more_than_64_kb_of_dynamic_lds_needs_the_function_attribute():
    """The GPU runtime refuses a launch with more than 64 KB of dynamic LDS unless hipFuncSetAttribute raised the
    kernel's limit first; so does the model (every large-LDS launch of the library goes through this check)."""
    m = Model()
    dst = _u32(m, 64)
    m.lib.simtest_big_lds(dst.p, 100 << 10, 0)
    assert any("bytes of dynamic LDS" in s and "65536" in s for s in m.violations()), m.violations()
    m.clear()
    m.lib.simtest_big_lds(dst.p, 64 << 10, 0)  # up to 64 KB need nothing
    m.lib.simtest_big_lds(dst.p, 100 << 10, 1)
    assert m.violations() == [] and (dst.get() == 0x5A).all()
    m.lib.simtest_big_lds(dst.p, 150 << 10, 0)  # allowed 100 KB so far
    assert any("allowed this kernel 102400" in s for s in m.violations()), m.violations()


@in_child
def test_execution_masks():
    m = Model()
    data = m.dev(np.arange(64, dtype=np.uint32))
    m.lib.simtest_exec_mask(data.p, 10, 1000, 1)
    assert m.violations() == []
    want = np.arange(64, dtype=np.uint32)
    want[:10] += 1000
    assert np.array_equal(data.get(), want)
    m.lib.simtest_exec_mask(data.p, 10, 1000, 0)
    assert any("execution mask other than" in s for s in m.violations()), m.violations()


@in_child
def test_lane_exchanges_against_the_instruction_definitions():
    m = Model()
    x = (np.arange(64, dtype=np.uint32) * 7 + 3)
    out = m.empty((17, 64), np.uint32)
    m.lib.simtest_lane_exchange(m.dev(x).p, out.p)
    assert m.violations() == []
    o = out.get()
    lane = np.arange(64)
    row, i = lane & ~15, lane & 15
    assert np.array_equal(o[0], x[lane ^ 1]) and np.array_equal(o[1], x[lane ^ 2])          # quad permutes
    assert np.array_equal(o[2], np.where(i + 4 < 16, x[np.minimum(lane + 4, 63)], 0xFFFFFFFF))  # row_shl:4 reads l + 4
    assert np.array_equal(o[3], np.where(i >= 4, x[np.maximum(lane - 4, 0)], 0xFFFFFFFF))       # row_shr:4 reads l - 4
    assert np.array_equal(o[4], x[row | ((i - 8) & 15)])                                      # row_ror:8
    assert np.array_equal(o[5], x[row | (15 - i)]) and np.array_equal(o[6], x[(lane & ~7) | (7 - (lane & 7))])
    # v_permlane16_swap: odd rows of the first operand <-> even rows of the second
    y = x + 1000
    odd = (lane // 16) % 2 == 1
    assert np.array_equal(o[7], np.where(odd, y[lane - 16 * odd], x))
    assert np.array_equal(o[8], np.where(~odd, x[np.minimum(lane + 16, 63)], y))
    # v_permlane32_swap: rows 2, 3 of the first operand <-> rows 0, 1 of the second
    hi = lane >= 32
    assert np.array_equal(o[9], np.where(hi, y[lane - 32 * hi], x))
    assert np.array_equal(o[10], np.where(~hi, x[np.minimum(lane + 32, 63)], y))
    assert np.all(o[11] == x[37]) and np.all(o[12] == x[0])
    ballot = sum(1 << int(l) for l in lane if x[l] & 1)
    assert np.all(o[13] == (ballot & 0xFFFFFFFF)) and np.all(o[14] == (ballot >> 32))
    assert np.array_equal(o[15], x[lane ^ 5])
    assert np.array_equal(o[16], np.where(lane >= 3, x[np.maximum(lane - 3, 0)], x))


@in_child
@pytest.mark.parametrize("asm_form", [0, 1])
def test_matrix_instruction_against_a_plain_matrix_product(asm_form):
    m = Model()
    rng = np.random.default_rng(5)
    a = f32_to_bf16_bits(rng.standard_normal((32, 16), dtype=np.float32))
    b = f32_to_bf16_bits(rng.standard_normal((16, 32), dtype=np.float32))
    c = rng.standard_normal((32, 32), dtype=np.float32)
    d = m.empty((32, 32), np.float32)
    m.lib.simtest_mfma(m.dev(a).p, m.dev(b).p, m.dev(c).p, d.p, asm_form)
    assert m.violations() == []
    want = bf16_bits_to_f32(a).astype(np.float64) @ bf16_bits_to_f32(b).astype(np.float64) + c
    assert np.allclose(d.get(), want, rtol=1e-6, atol=1e-6)
    # a one-hot B copies columns of A: exact
    b1 = np.zeros((16, 32), np.uint16)
    b1[3, 5] = b1[12, 17] = 0x3F80
    m.lib.simtest_mfma(m.dev(a).p, m.dev(b1).p, m.dev(np.zeros((32, 32), np.float32)).p, d.p, asm_form)
    got = d.get()
    assert np.array_equal(got[:, 5], bf16_bits_to_f32(a[:, 3])) and np.array_equal(got[:, 17], bf16_bits_to_f32(a[:, 12]))
    assert np.count_nonzero(got) == np.count_nonzero(a[:, 3]) + np.count_nonzero(a[:, 12])


@in_child
def test_meetings_barriers_and_spinning():
    m = Model()
    out, never = _u32(m, 128), m.dev(np.zeros(1, np.uint32))
    m.lib.simtest_meeting(out.p, never.p, 0)
    assert m.violations() == []
    assert np.array_equal(out.get(), np.repeat([22, 21], 64))  # multiples of 3 among the threads 0..63 and 64..127
    m.lib.simtest_meeting(out.p, never.p, 1)
    assert any("different wavefront-wide operations" in s for s in m.violations()), m.violations()
    m.clear()
    m.lib.simtest_meeting(out.p, never.p, 2)
    assert any("cannot go on" in s and "64 spinning" in s for s in m.violations()), m.violations()
    m.clear()
    for schedule in (0, 1, 99):
        m.lib.sim_set_schedule(schedule)
        m.lib.simtest_handover(out.p)
        assert m.violations() == [] and np.all(out.get()[:64] == 4711)


def test_a_plain_load_past_an_array_faults_and_names_the_kernel(capfd):
    @in_child
    def body():
        m = Model()
        src, dst = m.dev(np.zeros(1000, np.uint32)), _u32(m, 64)
        m.lib.simtest_plain_overrun(src.p, 1000, dst.p)

    with pytest.raises(AssertionError, match="memory fault inside the host model"):
        body()
    err = capfd.readouterr().err
    assert "st_plain_overrun_kernel" in err and "offset 4064" in err, err


def test_the_python_descriptor_matches_the_header():
    """ci_tiled_weight as tests/hostmodel/model.py declares it = the product's own ctypes declaration."""
    from comp_inference_amd import _lib
    from tests.hostmodel import model

    assert [(n, t) for n, t in model.TiledWeight._fields_] == [(n, t) for n, t in _lib.TiledWeight._fields_]
    assert C.sizeof(model.TiledWeight) == C.sizeof(_lib.TiledWeight)


def test_a_test_body_that_never_ends_is_ended(monkeypatch):
    """A kernel that loops for ever inside the model (nothing in it waits, so nothing reports a deadlock) must cost one
    test, not the test run: the child processes of the helpers have a time limit."""
    import time

    from tests.hostmodel import model

    monkeypatch.setattr(model, "CHILD_SECONDS", 1)
    with pytest.raises(AssertionError, match="did not finish within 1 s"):
        model.in_child(lambda: time.sleep(30))()
    with pytest.raises(AssertionError, match="did not finish within 2 s"):
        model.fork_all(lambda arg: time.sleep(30 if arg else 0), [0, 1])


# ---- the ordering check (the build with instrumented memory accesses) ------------------------------------------------
def _order_model():
    from tests.hostmodel import build

    m = Model(lib_path=build.build(order=True))
    assert m.lib.sim_checks_ordering() == 1
    return m


@in_child
def test_ordered_accesses_of_two_wavefronts_are_no_violation():
    """Writes, a barrier, the neighbour's reads, a barrier, writes again; a word handed over with release and acquire;
    every workgroup its own part of the output."""
    m = _order_model()
    out = _u32(m, 512)
    m.lib.simtest_ordering(out.p, 0)
    assert m.violations() == []
    tid = np.arange(256)
    want = ((tid // 64 + 1) % 4 * 64 + tid % 64) * 7 + np.where(tid < 64, 4711, 0)
    assert np.array_equal(out.get(), np.concatenate([want, want]))


@pytest.mark.parametrize("which, said", [
    (1, "of the LDS"),  # no barrier between the writes and the neighbour's reads
    (2, "of the LDS"),  # the second writes follow the neighbour's reads without a barrier
    (3, "of the LDS"),  # a flag without release / acquire orders nothing
    (4, "of the LDS"),  # a read of the assembly interpreter
    (5, "a __shared__ array"),
    (6, "overwrites byte"),  # two workgroups write the same words
    (7, "in the same launch"),  # a workgroup reads what another one writes
])
@in_child
def test_unordered_accesses_of_two_wavefronts_are_reported(which, said):
    m = _order_model()
    out = _u32(m, 512)
    m.lib.simtest_ordering(out.p, which)
    v = m.violations()
    assert v and all("ordering:" in s for s in v) and any(said in s for s in v), v


@in_child
def test_the_plain_build_does_not_check_ordering():
    m = Model()
    assert m.lib.sim_checks_ordering() == 0
    out = _u32(m, 512)
    m.lib.simtest_ordering(out.p, 1)
    assert m.violations() == []


@in_child
def test_a_read_of_bytes_that_nothing_has_written_is_reported():
    """The same build: a kernel that reads an array nobody has filled -- through an assembly statement and through
    plain C++ -- and the same reads after an upload."""
    m = _order_model()
    src, dst = m.empty(100, np.uint32), _u32(m, 64)
    m.lib.simtest_global_load(src.p, 50, dst.p, 0)
    v = m.violations()
    assert v and "nothing has written" in v[0], v
    m.clear()
    m.lib.simtest_plain_overrun(src.p, 10, dst.p)  # (words 26 .. 89 of the 100)
    v = m.violations()
    assert v and "nothing has written" in v[0], v
    m.clear()
    src.put(np.arange(100, dtype=np.uint32))
    m.lib.simtest_global_load(src.p, 50, dst.p, 0)
    m.lib.simtest_plain_overrun(src.p, 10, dst.p)
    assert m.violations() == [] and np.array_equal(dst.get(), 26 + np.arange(64))
    # what a kernel wrote is written: dst, read by the next launch
    out = _u32(m, 64)
    m.lib.simtest_global_load(dst.p, 64, out.p, 0)
    assert m.violations() == [] and np.array_equal(out.get(), 2 * (26 + np.arange(64)))


@in_child
def test_a_result_that_depends_on_the_order_of_the_lanes_is_reported():
    """A running sum through the LDS comes out right here, where lane l runs after lane l - 1, and would not on the GPU:
    the same build reports the pair of accesses."""
    m = _order_model()
    out = _u32(m, 64)
    m.lib.simtest_lane_order(out.p, 0)
    assert m.violations() == [] and np.array_equal(out.get(), 2 * np.arange(64) + 1)
    m.lib.simtest_lane_order(out.p, 1)
    v = m.violations()
    assert np.array_equal(out.get(), np.cumsum(np.arange(64) + 1))  # (lane order: the sum the GPU would not compute)
    assert v and "of the same wavefront wrote" in v[0] and "order in which the model runs the lanes" in v[0], v
    m.clear()
    m.lib.simtest_lane_order(out.p, 2)  # the same through an array
    v = m.violations()
    assert np.array_equal(out.get(), np.cumsum(np.arange(64) + 1))
    assert v and "of allocation" in v[0] and "of the same wavefront wrote" in v[0], v


# ---- the build with the compiler's undefined-behaviour checks ---------------------------------------------------------
def _undefined(which):
    from tests.hostmodel import build

    m = Model(lib_path=build.build(undefined=True))
    out = _u32(m, 64)
    m.lib.simtest_undefined(out.p, 0, 32)
    assert m.violations() == [] and np.array_equal(out.get(), np.arange(64) + np.arange(64) % 4)
    m.lib.simtest_undefined(out.p, which, 32)
    return m.violations()


@pytest.mark.parametrize("which, said", [(1, "shift_out_of_bounds"), (3, "type_mismatch"), (4, "add_overflow")])
@in_child
def test_undefined_behaviour_in_kernel_code_is_reported(which, said):
    v = _undefined(which)
    assert v and all("undefined behaviour" in s and "selftest.hip" in s for s in v) and said in v[0], v


def test_an_index_past_an_array_ends_the_run_and_says_where(capfd):
    """(What follows such an index is unreachable for the compiler: the model cannot go on and says so on stderr.)"""
    with pytest.raises(AssertionError, match="exited with 72"):
        in_child(_undefined)(2)
    assert "out_of_bounds at" in capfd.readouterr().err
