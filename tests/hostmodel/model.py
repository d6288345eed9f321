"""Python side of the host model: loads libci_hostmodel.so (the library's own sources compiled for the CPU model
of a gfx950 workgroup, tests/hostmodel/sim.h), hands it arrays that end at an inaccessible page, and reports what
the model saw.  numpy only.  Test infrastructure.
"""
from __future__ import annotations

import ctypes as C
import os
import pickle
import signal
import sys
import traceback

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

CI_SLOT_TABLE_BYTES = 32768


class TiledWeight(C.Structure):
    """ci_tiled_weight (include/comp_inference_hip.h)."""
    _fields_ = [("K", C.c_uint32), ("N", C.c_uint32), ("tile_height", C.c_uint32), ("tile_width", C.c_uint32),
                ("d_stream", C.c_void_p), ("stream_len", C.c_uint64),
                ("d_states", C.c_void_p), ("n_states", C.c_uint64),
                ("d_tables", C.c_void_p), ("d_slot_map", C.c_void_p),
                ("d_tile_offsets", C.c_void_p), ("d_tile_max_lens", C.c_void_p), ("n_tiles", C.c_uint64),
                ("d_man_tiled", C.c_void_p), ("man_len", C.c_uint64),
                ("d_checkpoints", C.c_void_p), ("checkpoint_bytes", C.c_uint64), ("segments", C.c_uint32),
                ("d_slot_table", C.c_void_p), ("slot_table_bytes", C.c_uint64), ("max_window_rows", C.c_uint32)]


class DecodeItem(C.Structure):
    """ci_decode_item."""
    _fields_ = [("d_stream", C.c_void_p), ("stream_len", C.c_uint64), ("d_states", C.c_void_p),
                ("d_tables", C.c_void_p), ("d_slot_map", C.c_void_p), ("d_tile_offsets", C.c_void_p),
                ("d_tile_max_lens", C.c_void_p), ("K", C.c_uint32), ("N", C.c_uint32), ("tile_height", C.c_uint32),
                ("tile_width", C.c_uint32), ("d_out_exp", C.c_void_p), ("d_checkpoints", C.c_void_p),
                ("segments", C.c_uint32)]


class Dev:
    """An array in the model's checked memory."""

    def __init__(self, ptr: int, shape, dtype, lib=None):
        self.ptr, self.shape, self.dtype, self.lib = ptr, tuple(shape), np.dtype(dtype), lib

    @property
    def nbytes(self) -> int:
        return int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize

    @property
    def p(self) -> C.c_void_p:
        return C.c_void_p(self.ptr if self.nbytes else 0)

    def get(self) -> np.ndarray:
        out = np.empty(self.shape, self.dtype)
        if self.nbytes:
            C.memmove(out.ctypes.data, self.ptr, self.nbytes)
        return out

    def put(self, values: np.ndarray) -> None:
        a = np.ascontiguousarray(values, self.dtype)
        assert a.size * a.itemsize == self.nbytes, (a.shape, self.shape)
        if self.nbytes:
            C.memmove(self.ptr, a.ctypes.data, self.nbytes)
            if self.lib is not None:  # (the build that checks it: a kernel may read what an upload wrote)
                self.lib.sim_mark_written(C.c_void_p(self.ptr), C.c_size_t(self.nbytes))


# a test body on the model takes seconds, a sweep block a minute or two
CHILD_SECONDS = 600


class ModelError(AssertionError):
    pass


class Model:
    def __init__(self, cus: int = 8, end_at_guard: bool = True, schedule: int = 0, lib_path: str | None = None):
        from tests.hostmodel import build

        # (lib_path, or CI_HOSTMODEL_LIB for a whole test run: a build with a deliberate mistake, build.build_mutant)
        self.lib = C.CDLL(lib_path or os.environ.get("CI_HOSTMODEL_LIB") or build.build())
        L = self.lib
        L.sim_alloc.restype = C.c_void_p
        L.sim_alloc.argtypes = [C.c_size_t, C.c_int]
        L.sim_violation.restype = C.c_char_p
        L.sim_launch_name.restype = C.c_char_p
        L.sim_asm_instructions.restype = C.c_uint64
        L.ci_last_error.restype = C.c_char_p
        for f in ("ci_encode_scratch_bytes", "ci_fused_linear_workspace_bytes", "ci_fused_embedding_workspace_bytes",
                  "ci_fused_linear_transposed_workspace_bytes", "ci_fused_linear_workspace_bytes_segmented",
                  "ci_checkpoint_bytes", "ci_fused_embedding_workspace_bytes_segmented"):
            getattr(L, f).restype = C.c_size_t
        L.ci_suggest_segments.restype = C.c_uint32
        L.sim_init()
        L.sim_set_cus(cus)
        L.sim_set_schedule.argtypes = [C.c_uint64]
        L.sim_set_schedule(schedule)
        self.end_at_guard = 1 if end_at_guard else 0
        L.sim_free_all()
        L.sim_clear()

    # ---- memory
    def dev(self, a: np.ndarray) -> Dev:
        a = np.ascontiguousarray(a)
        d = self.empty(a.shape, a.dtype)
        d.put(a)
        return d

    def empty(self, shape, dtype) -> Dev:
        shape = (shape,) if np.isscalar(shape) else tuple(shape)
        n = int(np.prod(shape, dtype=np.int64)) * np.dtype(dtype).itemsize
        ptr = self.lib.sim_alloc(n, self.end_at_guard)
        assert ptr, "sim_alloc failed"
        return Dev(ptr, shape, dtype, self.lib)

    def free_all(self) -> None:
        self.lib.sim_free_all()

    # ---- calls
    def call(self, name: str, *args) -> None:
        """Run an entry point; raise if it reports an error or the model saw a violation."""
        rc = getattr(self.lib, name)(*args)
        viol = self.violations()
        if viol:
            self.lib.sim_clear()
            raise ModelError(f"{name}: " + "\n  ".join(viol[:8]))
        if rc != 0:
            raise RuntimeError(f"{name}: rc {rc}: {self.lib.ci_last_error().decode()}")

    def violations(self) -> list[str]:
        return [self.lib.sim_violation(i).decode() for i in range(self.lib.sim_violation_count())]

    def asm_instructions(self) -> int:
        """Instructions of hand-written assembly statements the interpreter has carried out so far (per wavefront)."""
        return int(self.lib.sim_asm_instructions())

    def launches(self) -> list[str]:
        return [self.lib.sim_launch_name(i).decode() for i in range(self.lib.sim_launch_count())]

    def clear(self) -> None:
        self.lib.sim_clear()

    # ---- a compressed weight as the entry points take it
    def weight(self, enc, man_tiled, K: int, N: int, segments: int = 1, slot_table: bool = False,
               window_rows: bool = False):
        """ci_tiled_weight over copies of the oracle's arrays (and what keeps them alive).  `segments` > 1 builds
        the decoder checkpoints with the library, `slot_table` the 32 KB table, `window_rows` the largest window."""
        keep = dict(stream=self.dev(enc.stream), states=self.dev(enc.states), tables=self.dev(enc.tables),
                    slot_map=self.dev(enc.slot_map), offs=self.dev(enc.tile_offsets), lens=self.dev(enc.tile_max_lens))
        w = TiledWeight()
        w.K, w.N, w.tile_height, w.tile_width = K, N, enc.tile_height, enc.tile_width
        w.d_stream, w.stream_len = keep["stream"].p, enc.stream.size
        w.d_states, w.n_states = keep["states"].p, enc.states.size
        w.d_tables, w.d_slot_map = keep["tables"].p, keep["slot_map"].p
        w.d_tile_offsets, w.d_tile_max_lens, w.n_tiles = keep["offs"].p, keep["lens"].p, enc.tile_offsets.size
        if man_tiled is not None:
            keep["man"] = self.dev(man_tiled)
            w.d_man_tiled, w.man_len = keep["man"].p, man_tiled.size
        w.segments = 1
        if segments > 1:
            nb = self.lib.ci_checkpoint_bytes(K, N, enc.tile_height, enc.tile_width, segments)
            keep["ckpt"] = self.empty(nb // 8 * 2, np.uint32)
            # (pointers go in as c_void_p objects: a plain int would be passed as a 32-bit C int)
            self.call("ci_build_checkpoints_ilp2", keep["stream"].p, C.c_uint64(w.stream_len), keep["states"].p,
                      keep["tables"].p, keep["slot_map"].p, keep["offs"].p, keep["lens"].p, K, N, enc.tile_height,
                      enc.tile_width, segments, keep["ckpt"].p, C.c_size_t(nb), None)
            w.d_checkpoints, w.checkpoint_bytes, w.segments = keep["ckpt"].p, nb, segments
        if slot_table:
            keep["slot_table"] = self.empty(CI_SLOT_TABLE_BYTES // 4, np.uint32)
            self.call("ci_build_slot_table", keep["tables"].p, keep["slot_map"].p, keep["slot_table"].p, C.c_size_t(CI_SLOT_TABLE_BYTES), None)
            w.d_slot_table, w.slot_table_bytes = keep["slot_table"].p, CI_SLOT_TABLE_BYTES
        if window_rows:
            keep["rows"] = self.empty(1, np.uint32)
            self.call("ci_max_window_rows", C.byref(w), keep["rows"].p, None)
            w.max_window_rows = int(keep["rows"].get()[0])
        return w, keep


# ---- synthetic inputs (the recipes of tests/helpers.py without torch) ---------------------------------------------
def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def weight_bits(K: int, N: int, seed: int, std: float = 0.02) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return f32_to_bf16_bits((rng.standard_normal((K, N), dtype=np.float32) * std))


def x_bits(M: int, K: int, seed: int) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return f32_to_bf16_bits(rng.standard_normal((M, K), dtype=np.float32))


# ---- running a test body in a child process -----------------------------------------------------------------------
def in_child(fn):
    """Decorator: the test body runs in a forked child, so that a memory fault inside the model (which ends the
    process with a message naming kernel, workgroup, thread and address) fails one test and not the test run."""
    import functools

    @functools.wraps(fn)
    def wrapper(*args, **kwargs):
        r, w = os.pipe()
        sys.stdout.flush()
        sys.stderr.flush()
        pid = os.fork()
        if pid == 0:
            os.close(r)
            code = 0
            signal.alarm(CHILD_SECONDS)  # (a kernel that loops for ever in the model ends its child, not the test run)
            # The oracle is OpenMP code, and a process forked from one whose OpenMP runtime already has its worker
            # threads (an earlier test used the oracle) would wait for those threads for ever: teams of one here.
            try:
                C.CDLL("libgomp.so.1").omp_set_num_threads(1)
            except OSError:
                pass
            try:
                fn(*args, **kwargs)
                payload = pickle.dumps(None)
            except BaseException:  # noqa: BLE001
                payload = pickle.dumps(traceback.format_exc())
                code = 1
            with os.fdopen(w, "wb") as f:
                f.write(payload)
            sys.stdout.flush()
            sys.stderr.flush()
            os._exit(code)
        os.close(w)
        with os.fdopen(r, "rb") as f:
            data = f.read()
        _, status = os.waitpid(pid, 0)
        if os.WIFSIGNALED(status) and os.WTERMSIG(status) == signal.SIGALRM:
            raise AssertionError(f"the host model did not finish within {CHILD_SECONDS} s: a kernel that loops for ever?")
        if os.WIFSIGNALED(status):
            raise AssertionError(f"the host-model child died of signal {os.WTERMSIG(status)}")
        code = os.WEXITSTATUS(status)
        if code == 70:
            raise AssertionError("memory fault inside the host model (see the message on stderr)")
        err = pickle.loads(data) if data else f"child exited with {code} and no report"
        if err is not None:
            raise AssertionError(err)

    return wrapper


def in_fresh_process(fn):
    """Like in_child, but the body runs in a new interpreter (the oracle keeps all its threads there): for the few
    tests whose inputs take the oracle tens of seconds to encode.  The test function must be a module-level one
    whose arguments have a repr that evaluates to them."""
    import functools
    import subprocess

    @functools.wraps(fn)
    def wrapper(*args, **kwargs):
        code = (f"import sys; sys.path[:0] = [{ROOT!r}, {os.path.join(ROOT, 'tests')!r}]; import importlib; "
                f"f = getattr(importlib.import_module({fn.__module__.split('.')[-1]!r}), {fn.__name__!r}); "
                f"f.__wrapped__(*{args!r}, **{kwargs!r})")
        try:
            p = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=2 * CHILD_SECONDS)
        except subprocess.TimeoutExpired:
            raise AssertionError(f"the host model did not finish within {2 * CHILD_SECONDS} s: a kernel that loops for ever?") from None
        sys.stderr.write(p.stderr[-4000:])
        if p.returncode == 70:
            raise AssertionError("memory fault inside the host model:\n" + p.stderr[-2000:])
        if p.returncode != 0:
            raise AssertionError(p.stderr[-6000:] or f"child exited with {p.returncode}")

    return wrapper


def fork_all(fn, arg_list, jobs: int | None = None):
    """fn(arg) for every arg, each in a forked child (see in_child), up to `jobs` at a time; raises AssertionError with
    every failure's report.  The children write nothing but their report."""
    jobs = jobs or max(1, (os.cpu_count() or 2) - 1)
    pending, running, failures = list(arg_list), {}, []
    from tests.hostmodel import build

    build.build()  # once, here: children that each found the library out of date would all write it at the same time

    def start(arg):
        r, w = os.pipe()
        sys.stdout.flush()
        sys.stderr.flush()
        pid = os.fork()
        if pid == 0:
            os.close(r)
            code = 0
            signal.alarm(2 * CHILD_SECONDS)
            try:
                C.CDLL("libgomp.so.1").omp_set_num_threads(1)  # (see in_child)
            except OSError:
                pass
            try:
                fn(arg)
                payload = pickle.dumps(None)
            except BaseException:  # noqa: BLE001
                payload = pickle.dumps(traceback.format_exc())
                code = 1
            with os.fdopen(w, "wb") as f:
                f.write(payload)
            sys.stdout.flush()
            sys.stderr.flush()
            os._exit(code)
        os.close(w)
        running[pid] = (arg, r)

    while pending or running:
        while pending and len(running) < jobs:
            start(pending.pop(0))
        pid, status = os.wait()
        if pid not in running:
            continue
        arg, r = running.pop(pid)
        with os.fdopen(r, "rb") as f:
            data = f.read()
        if os.WIFSIGNALED(status) and os.WTERMSIG(status) == signal.SIGALRM:
            failures.append(f"[{arg!r}] the host model did not finish within {2 * CHILD_SECONDS} s: a kernel that loops for ever?")
        elif os.WIFSIGNALED(status):
            failures.append(f"[{arg!r}] the child died of signal {os.WTERMSIG(status)}")
        elif os.WEXITSTATUS(status) == 70:
            failures.append(f"[{arg!r}] memory fault inside the host model (see the message on stderr)")
        else:
            err = pickle.loads(data) if data else f"child exited with {os.WEXITSTATUS(status)} and no report"
            if err is not None:
                failures.append(f"[{arg!r}] {err}")
    if failures:
        raise AssertionError("\n".join(failures))
