#!/usr/bin/env python3
"""Benchmark of the compressed-weight hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (one "step"): stand-alone rANS decode of the seven weight tensors of one
Llama-3-8B-shaped decoder layer (q, k, v, o, gate, up, down), bf16 N(0, 0.02) from seed 1,
default format (1024x32 tiles, two streams per column, 12-bit per-tensor table).  All inputs are
resident in HBM before the timed region.  `value` = exponent-plane bytes decoded per second.

The JSON line also carries
  roofline      decode kernel, algorithmic bytes per launch / measured launch time vs 8 TB/s HBM
  cpu_baseline  the CPU oracle decoding the same streams on the host cores (bounded sample)
  fused_gemv    fused decompress-GEMV/GEMM on the gate projection for M = 1, 4, 16, 64:
                time, share of the HBM roofline on compressed bytes, and torch.matmul (hipBLASLt)
                on the uncompressed bf16 weight for comparison
  fused_gemv_layer_M1, fused_embedding, lm_head   the other operators at their full sizes
  fused_model   batch-1 greedy decode of a 32-layer Llama-3-8B-shaped decoder on compressed weights
                (bench_model.run), tok/s next to the same decoder on bf16 weights
  cpu_roundtrip one 4096x4096 tensor (seed 0) through the CPU oracle's encoder and decoder
Every fraction of the HBM peak in the line is repeated in roofline.kernels with the bytes and the time
it was computed from.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# The binding limit of byte-wise rANS on this chip is not HBM but the rate of dependent decode steps:
# one step of one wavefront (64 streams) takes about 6.0 ns of a CU that sixteen wavefronts share (one
# random 8-byte table read and one byte read from LDS, eight VALU instructions), and a lone wavefront needs
# about 87 ns per step (profiles/step_rate_microbench.md).  Reported next to every HBM fraction.
STEP_NS_PER_CU = 6.0
STEP_NS_LATENCY = 87.0
NUM_CUS = 256  # replaced by the device's own count in main()


# Two floors no schedule gets under, from what the step is made of: ten VALU instructions of 64 lanes on four 16-lane SIMDs
# at 2.4 GHz (the chip's 39 T integer lane-operations a second) are 4.17 ns of a CU per wavefront-step, and the LDS
# pipe needs 2.64 + 1.95 ns for the step's random 8-byte table read and its byte read (the same microbenchmark).
STEP_VALU_INSTRUCTIONS = 10
STEP_NS_VALU_FLOOR = STEP_VALU_INSTRUCTIONS * 64 / (4 * 16 * 2.4)  # ns of one CU
STEP_NS_LDS_FLOOR = 2.64 + 1.95


def step_bound_us(wave_steps: int, chain: int) -> dict:
    """Lower bounds from the step rate: throughput (all CUs busy) at the measured rate and at the step's VALU-issue and
    LDS-pipe floors, and latency (one chain)."""
    return {"throughput_us": round(wave_steps * STEP_NS_PER_CU / NUM_CUS * 1e-3, 1),
            "valu_issue_floor_us": round(wave_steps * STEP_NS_VALU_FLOOR / NUM_CUS * 1e-3, 1),
            "lds_pipe_floor_us": round(wave_steps * STEP_NS_LDS_FLOOR / NUM_CUS * 1e-3, 1),
            "latency_us": round(chain * STEP_NS_LATENCY * 1e-3, 1)}
# HBM bytes of one batched decode launch on this workload are not measured by this program: they come from two
# rocprofv3 counter passes over this same command (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), each scaled by what
# the same counter reads for a plain copy of known size (--copy-calibration).  `bench.py --record-traffic FETCH.csv
# WRITE.csv` turns the two counter files into profiles/traffic.json, which also holds a digest of the kernel sources
# it was taken on; a run reports the figure only while the sources are still those, and null otherwise.
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "traffic.json")
TRAFFIC_KERNEL = "decode_tiled32_seg_kernel"
COPY_KERNEL, COPY_BYTES = "__amd_rocclr_copyBuffer", 64 << 20  # what --copy-calibration launches


def sources_digest() -> str:
    """sha256 over the kernel sources (names and contents): what a counter figure was measured on."""
    import hashlib

    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "comp_inference_amd", "csrc")
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".hip", ".h")):
            h.update(name.encode())
            with open(os.path.join(csrc, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()[:16]


def _counter_kib(csv_path: str, counter: str, kernel: str, first: int = 0) -> float:
    """Mean of `counter` over the dispatches of the kernels whose name contains `kernel` (rocprofv3 --pmc, csv);
    `first` > 0: over the first so many of them only."""
    import csv

    vals = []
    with open(csv_path, newline="") as f:
        for row in csv.DictReader(f):
            if row["Counter_Name"] == counter and kernel in row["Kernel_Name"]:
                vals.append((int(row["Dispatch_Id"]), float(row["Counter_Value"])))
    if not vals:
        raise SystemExit(f"{csv_path}: no {counter} reading for a kernel named *{kernel}*")
    vals = [v for _, v in sorted(vals)][:first or None]
    return sum(vals) / len(vals)


def record_traffic(fetch_csv: str, write_csv: str) -> int:
    """profiles/traffic.json from the two counter files (no GPU needed)."""
    fetch, write = _counter_kib(fetch_csv, "FETCH_SIZE", TRAFFIC_KERNEL), _counter_kib(write_csv, "WRITE_SIZE", TRAFFIC_KERNEL)
    # (the calibration copies are the first three copies of the run: --copy-calibration runs before anything is uploaded)
    f_scale = COPY_BYTES / 1024 / _counter_kib(fetch_csv, "FETCH_SIZE", COPY_KERNEL, first=3)
    w_scale = COPY_BYTES / 1024 / _counter_kib(write_csv, "WRITE_SIZE", COPY_KERNEL, first=3)
    rec = {"kernel": TRAFFIC_KERNEL, "workload": "llama3-8b layer, seven tensors, one launch, 2 segments per stream",
           "fetch_kib": round(fetch, 1), "fetch_scale": round(f_scale, 4), "write_kib": round(write, 1),
           "write_scale": round(w_scale, 4), "bytes": int(round((fetch * f_scale + write * w_scale) * 1024)),
           "sources": sources_digest(),
           "command": "rocprofv3 --pmc FETCH_SIZE (then WRITE_SIZE) --output-format csv -- python3 bench.py --steps 3 --warmup 1 "
                      "--no-cpu-baseline --no-gemv --no-embedding --no-model --copy-calibration"}
    with open(TRAFFIC_JSON, "w") as f:
        json.dump(rec, f, indent=1)
        f.write("\n")
    print(json.dumps(rec))
    return 0


def measured_traffic():
    """(bytes or None, where the answer comes from)."""
    try:
        with open(TRAFFIC_JSON) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None, "no counter record (profiles/traffic.json)"
    now = sources_digest()
    if rec.get("sources") != now or rec.get("kernel") != TRAFFIC_KERNEL:
        return None, (f"profiles/traffic.json holds {rec.get('bytes')} bytes measured on kernel sources {rec.get('sources')}; "
                      f"the sources are now {now}: not carried over")
    return int(rec["bytes"]), "profiles/traffic.json (offline rocprofv3 counter passes over this command on these sources)"


LAYER = [("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096),
         ("gate", 14336, 4096), ("up", 14336, 4096), ("down", 4096, 14336)]  # (name, out, in)


# the other workloads of the line (module constants so that a rehearsal of this file can run them small)
GEMV_ROWS = (1, 4, 16, 64)
GEMM_ROWS = (16, 64, 128, 256, 512, 2048, 8192)
EMBED_SHAPE = (128256, 4096, 2048)  # table rows, columns, ids


def log(msg: str) -> None:
    print(msg, file=sys.stderr, flush=True)


def make_layer(seed: int):
    """Weights drawn in the listed order from one generator, nn.Linear orientation [out, in]."""
    g = torch.Generator("cpu").manual_seed(seed)
    return [(name, (torch.randn(o, i, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16))
            for name, o, i in LAYER]


class Compressed:
    """One weight in the default format, resident on the GPU."""

    def __init__(self, name: str, w_out_in: torch.Tensor, dev, th: int = 1024, tw: int = 32, transpose: bool = True):
        import comp_inference_amd as ci

        # linear weights are encoded as [K, N] = [in, out]; an embedding table as it is
        w = w_out_in.t().contiguous() if transpose else w_out_in.contiguous()
        self.name, self.K, self.N, self.th, self.tw = name, w.shape[0], w.shape[1], th, tw
        exp, man = ci.extract_exp_and_mantissa(w)
        f, c = ci.get_rans_lut(exp)
        r = ci.ccore.RansManager(exp.numel()).compress_tiled(exp, f, c, th, tw)
        self.host = r
        self.exp_host = exp.numpy()
        self.stream = r.stream.to(dev)
        self.states = r.states.to(dev)
        self.tables = r.tables.to(dev)
        self.slot_map = r.slot_map.to(dev)
        self.tile_offsets = r.tile_offsets.to(dev)
        self.tile_max_lens = r.tile_max_lens.to(dev)
        self.man = ci.interleave_mantissas(man, th, tw).to(dev)
        self.n_streams = r.num_streams
        self.n_tiles = r.num_tiles_k * r.num_tiles_n

    # algorithmic bytes of one stand-alone decode: stream + states + per-tile metadata + tables in,
    # exponent plane out
    def decode_bytes(self) -> int:
        return self.stream.numel() + 4 * self.n_streams + 8 * self.n_tiles + 1024 + 4096 + self.K * self.N

    # decode steps of 64 streams at a time (one wavefront-step): a tile is th/2 of them
    def wave_steps(self) -> int:
        return self.n_tiles * (self.th // 2)

    # algorithmic bytes of one fused linear at M rows
    def linear_bytes(self, M: int) -> int:
        return (self.stream.numel() + self.man.numel() + 4 * self.n_streams + 8 * self.n_tiles + 5120
                + 2 * M * self.K + 2 * M * self.N)

    def decode(self):
        import comp_inference_amd as ci

        return ci.rans_decomp_tiled(self.stream, self.states, self.tables, self.slot_map, (self.K, self.N),
                                    self.tile_offsets, self.tile_max_lens, tile_k=self.th, tile_n=self.tw)

    def linear(self, x):
        import comp_inference_amd as ci

        return ci.fused_rans_linear(x, self.stream, self.states, self.tables, self.slot_map, (self.K, self.N),
                                    self.tile_offsets, self.tile_max_lens, self.th, self.tw, self.man)

    def linear_segmented(self, x):
        """The fused linear with decoder checkpoints, as many segments as the library suggests for the shape
        (built once, on first use, like RansLinear does)."""
        import comp_inference_amd as ci

        if not hasattr(self, "segments"):
            from comp_inference_amd.linear_hip import PreparedLinear

            self.segments = ci.suggest_segments((self.K, self.N), self.th, self.tw)
            self.checkpoints = ci.build_checkpoints(self.stream, self.states, self.tables, self.slot_map,
                                                    (self.K, self.N), self.tile_offsets, self.tile_max_lens,
                                                    self.th, self.tw, self.segments)
            self.prepared = PreparedLinear(self.stream.device, self.stream, self.states, self.tables, self.slot_map,
                                           (self.K, self.N), self.tile_offsets, self.tile_max_lens, self.th, self.tw,
                                           self.man, checkpoints=self.checkpoints, segments=self.segments)
        return self.prepared(x)


def event_times_us(fn, warmup: int, iters: int):
    """Per-call GPU time with events on the stream the kernels are launched on."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    out = []
    for _ in range(iters):
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        fn()
        e.record()
        e.synchronize()
        out.append(s.elapsed_time(e) * 1e3)
    return out


def batched_time_us(fn, warmup: int, iters: int) -> float:
    """Average GPU time per call with `iters` calls enqueued back to back between two events, so
    that host launch latency is not part of the figure."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    e.synchronize()
    return s.elapsed_time(e) * 1e3 / iters


def cpu_baseline(layer: list[Compressed], budget_s: float = 15.0):
    """CPU oracle decoding the same streams, all host cores (OpenMP), median of repeated passes
    over the whole layer within a time budget."""
    from oracle import rans_oracle as ro

    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else os.cpu_count()
    cores = min(cores or 1, int(os.environ.get("OMP_NUM_THREADS", cores or 1)))
    args = [(c.host.stream.numpy(), c.host.states.view(torch.int32).numpy().view(np.uint32),
             c.host.tables.view(torch.int32).numpy().view(np.uint32), c.host.slot_map.numpy(),
             c.host.tile_offsets.view(torch.int32).numpy().view(np.uint32),
             c.host.tile_max_lens.view(torch.int32).numpy().view(np.uint32), c.K, c.N, c.th, c.tw) for c in layer]
    total = sum(c.K * c.N for c in layer)
    times = []
    t_start = time.time()
    checked = False
    while len(times) < 13 and (time.time() - t_start < budget_s or len(times) < 3):
        t0 = time.time()
        outs = [ro.decode_tiled_ilp2(*a) for a in args]
        times.append(time.time() - t0)
        if not checked:  # the baseline must be decoding the right thing
            assert all(np.array_equal(o, c.exp_host) for o, c in zip(outs, layer))
            checked = True
    med = float(np.median(times[1:])) if len(times) > 1 else times[0]
    # the CPU route to one GEMV on the gate projection: decode, join the planes, torch.matmul (all cores)
    gate = next(c for c in layer if c.name == "gate")
    ga = args[[c.name for c in layer].index("gate")]
    t0 = time.time()
    e = ro.decode_tiled_ilp2(*ga)
    t_dec = time.time() - t0
    man = ci_uninterleave(gate)
    t0 = time.time()
    w = torch.from_numpy(ro.merge_bf16(e, man).view(np.int16)).view(torch.bfloat16)
    t_merge = time.time() - t0
    x = torch.randn(1, gate.K, generator=torch.Generator("cpu").manual_seed(2)).to(torch.bfloat16)
    torch.set_num_threads(int(cores))
    torch.matmul(x, w)
    t0 = time.time()
    for _ in range(3):
        torch.matmul(x, w)
    t_mm = (time.time() - t0) / 3
    return {"value": round(total / med / 1e9, 3), "unit": "GB/s", "cores": int(cores), "kind": "port",
            "sample": f"whole layer ({total / 1e6:.0f} M symbols), {len(times)} passes, median, OpenMP over tiles",
            "gate_gemv_M1_ms": {"decode": round(t_dec * 1e3, 2), "merge_planes": round(t_merge * 1e3, 2),
                                "torch_matmul_bf16": round(t_mm * 1e3, 2)}}


def cpu_roundtrip(seed: int = 0, n: int = 4096):
    """One n x n bf16 tensor, N(0, 0.02) from `seed`, through the CPU oracle alone: planes split, exponent
    plane rANS-coded in the default tiling, decoded and joined again; bit-exact check, whole-tensor
    compression ratio and decode rate on the host cores."""
    from oracle import rans_oracle as ro

    g = torch.Generator("cpu").manual_seed(seed)
    w = (torch.randn(n, n, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16)
    bits = w.view(torch.int16).numpy().view(np.uint16)
    t0 = time.time()
    enc, man = ro.compress_bf16(bits, 1024, 32)
    t_enc = time.time() - t0
    dec_args = (enc.stream, enc.states, enc.tables, enc.slot_map, enc.tile_offsets, enc.tile_max_lens, n, n, 1024, 32)
    times = []
    for _ in range(5):
        t0 = time.time()
        e = ro.decode_tiled_ilp2(*dec_args)
        times.append(time.time() - t0)
    t_dec = float(np.median(times))
    back = ro.merge_bf16(e, ro.uninterleave_plane(man, n, n, 1024, 32))
    stored = enc.stream.size + man.size + 4 * enc.states.size + 4 * enc.tile_offsets.size + 4 * enc.tile_max_lens.size + 5120
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else os.cpu_count()
    cores = min(cores or 1, int(os.environ.get("OMP_NUM_THREADS", cores or 1)))
    return {"tensor": f"{n}x{n} bf16 N(0,0.02) seed {seed}, tile 1024x32", "bit_exact": bool(np.array_equal(back, bits)),
            "compression_ratio": round(2.0 * n * n / stored, 4),
            "exponent_plane_ratio": round(n * n / enc.stream.size, 4),
            "cpu_decode_GBs_exponent_bytes": round(n * n / t_dec / 1e9, 3),
            "cpu_decode_GBs_bf16_bytes": round(2.0 * n * n / t_dec / 1e9, 3),
            "cpu_encode_s": round(t_enc, 3), "cores": int(cores), "kind": "port"}


def ci_uninterleave(c: "Compressed") -> np.ndarray:
    """Row-major sign|mantissa plane of a compressed tensor (host)."""
    import comp_inference_amd as ci

    return ci.uninterleave_mantissas(c.man.cpu(), c.K, c.N, c.th, c.tw).numpy()


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-gemv", action="store_true")
    ap.add_argument("--no-embedding", action="store_true")
    ap.add_argument("--no-model", action="store_true", help="skip the 32-layer decoder (about a minute)")
    ap.add_argument("--new-kernels", action="store_true",
                    help="also time the kernels that are off by default (more than 64 rows of x in one pass, the "
                         "gather on sixteen wavefronts), each checked against the default path first")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three 64 MiB device-to-device copies, so that a counter run has a "
                         "kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    ap.add_argument("--record-traffic", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no benchmark: write profiles/traffic.json from the counter_collection.csv files of a FETCH_SIZE "
                         "and a WRITE_SIZE pass of rocprofv3 over `bench.py --copy-calibration`")
    a = ap.parse_args()
    if a.record_traffic:
        return record_traffic(*a.record_traffic)
    if a.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU part (run with --gpus 1)", file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (gfx950)", file=sys.stderr)
        return 2

    import comp_inference_amd as ci  # noqa: F401  (fails loudly if the HIP library is missing)

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    global NUM_CUS
    NUM_CUS = torch.cuda.get_device_properties(dev).multi_processor_count
    kernels = []  # every HBM fraction of the line with the bytes and the time behind it

    def record(kernel: str, config: str, nbytes: int, us: float) -> float:
        frac = nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS
        kernels.append({"kernel": kernel, "config": config, "bytes": int(nbytes), "us": round(us, 2), "frac": round(frac, 4)})
        return frac

    if a.copy_calibration:
        src = torch.full((64 << 20,), 7, device=dev, dtype=torch.uint8)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    log("generating and compressing one layer (seed 1) ...")
    layer = [Compressed(n, w, dev) for n, w in make_layer(1)]
    total_syms = sum(c.K * c.N for c in layer)
    total_stream = sum(c.stream.numel() for c in layer)

    # bit-exact check of what is about to be timed
    for c in layer:
        assert np.array_equal(c.decode().cpu().numpy(), c.exp_host), f"decode mismatch on {c.name}"

    plain_items = [(c.stream, c.states, c.tables, c.slot_map, (c.K, c.N), c.tile_offsets, c.tile_max_lens) for c in layer]
    th, tw = layer[0].th, layer[0].tw
    # decoder checkpoints: the decoder's state and position in the middle of every stream (an index of 8 bytes per
    # stream and checkpoint beside the compressed tensor, derived from it once; the stream itself is unchanged).
    # With them an item is half a stream and its window of the tile body fits sixteen wavefronts on a CU.
    DECODE_SEGMENTS = 2
    items = [it + (ci.build_checkpoints(*it, th, tw, DECODE_SEGMENTS), DECODE_SEGMENTS) for it in plain_items]
    checkpoint_bytes = sum(int(it[7].numel()) * 8 for it in items)

    # one step = the whole layer decoded by one batched launch (every tensor, every tile)
    def step():
        return ci.rans_decomp_tiled_batch(items, tile_k=th, tile_n=tw)

    for o, c in zip(step(), layer):
        assert np.array_equal(o.cpu().numpy(), c.exp_host), f"batched decode mismatch on {c.name}"

    # --- timed region: W warm-up steps, then exactly K steps between two synchronisations
    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()  # on the current stream, which is the stream the library launches on
    for _ in range(a.steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / a.steps
    launch_us = ev0.elapsed_time(ev1) * 1e3 / a.steps  # one decode launch per step, back to back
    value = total_syms / (ms_per_step * 1e-3) / 1e9

    # --- decode kernel roofline: per-launch durations by events on the launch stream
    per_kernel = {}
    for c in layer:
        per_kernel[c.name] = round(float(np.median(event_times_us(c.decode, 5, 30))), 2)
    algo_bytes = sum(c.decode_bytes() for c in layer) + checkpoint_bytes
    achieved = algo_bytes / (launch_us * 1e-6) / 1e9
    for o, c in zip(ci.rans_decomp_tiled_batch(plain_items, tile_k=th, tile_n=tw), layer):
        assert np.array_equal(o.cpu().numpy(), c.exp_host), f"decode without checkpoints: mismatch on {c.name}"
    us_whole_streams = batched_time_us(lambda: ci.rans_decomp_tiled_batch(plain_items, tile_k=th, tile_n=tw), 5, 20)
    traffic_bytes, traffic_source = measured_traffic()
    roofline = {"bound": "hbm", "kernel": "decode_tiled32_seg_kernel", "achieved": round(achieved, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": traffic_bytes, "traffic_source": traffic_source,
                "bytes_per_launch": int(algo_bytes), "cus": int(NUM_CUS),
                "launch_us": round(launch_us, 2), "single_tensor_launch_us": per_kernel,
                "decoder_checkpoint_segments": DECODE_SEGMENTS, "checkpoint_bytes": checkpoint_bytes,
                "launch_us_whole_streams_no_checkpoints": round(us_whole_streams, 2),
                "compressed_read_GBs": round(total_stream / (launch_us * 1e-6) / 1e9, 1)}
    record("decode_tiled32_seg_kernel", "one layer, seven tensors, one launch, 2 segments per stream", algo_bytes, launch_us)
    record("decode_tiled32_persist_kernel", "the same without checkpoints (whole streams)", algo_bytes - checkpoint_bytes, us_whole_streams)
    wave_steps = sum(c.wave_steps() for c in layer)
    sb = step_bound_us(wave_steps, th // 2 // DECODE_SEGMENTS)
    roofline["step_rate_bound"] = dict(sb, wavefront_steps=wave_steps, ns_per_wavefront_step_per_cu=STEP_NS_PER_CU,
                                       frac=round(sb["throughput_us"] / launch_us, 3))

    out = {"metric": "decoded GB/s", "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": a.steps,
           "warmup": a.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": "u8", "data": "synthetic",
           "config": {"workload": "standalone rANS decode of one Llama-3-8B-shaped layer (q,k,v,o,gate,up,down), "
                                  "bf16 N(0,0.02) seed 1, tile 1024x32, two streams per column, 12-bit tables, "
                                  "decoder checkpoints at the middle of every stream",
                      "symbols_per_step": total_syms, "compressed_stream_bytes": total_stream,
                      "exponent_plane_ratio": round(total_syms / total_stream, 3)},
           "roofline": roofline}

    # --- fused decompress-GEMV/GEMM on the gate projection
    if not a.no_gemv:
        gate = next(c for c in layer if c.name == "gate")
        g = torch.Generator("cpu").manual_seed(2)
        x_all = torch.randn(max(GEMV_ROWS), gate.K, generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev)
        w_dense = ci.rans_decomp_tiled(gate.stream, gate.states, gate.tables, gate.slot_map, (gate.K, gate.N),
                                       gate.tile_offsets, gate.tile_max_lens, mantissas=gate.man)
        rows = []
        for M in GEMV_ROWS:
            x = x_all[:M].contiguous()
            got = gate.linear_segmented(x).float()
            want = torch.matmul(x, w_dense).float()
            ok = bool(torch.allclose(got, want, atol=1e-2, rtol=1e-2))
            us = batched_time_us(lambda: gate.linear_segmented(x), 25, 100)
            us_plain = batched_time_us(lambda: gate.linear(x), 25, 100)
            us_ref = batched_time_us(lambda: torch.matmul(x, w_dense), 25, 100)
            nbytes = gate.linear_bytes(M)
            record("fused linear (checkpoints)", f"gate K={gate.K} N={gate.N} M={M}", nbytes, us)
            sb = step_bound_us(gate.wave_steps(), gate.th // 2 // int(gate.segments))
            rows.append({"M": M, "us": round(us, 2), "us_without_checkpoints": round(us_plain, 2), "allclose_1e-2": ok,
                         "step_rate_bound_us": max(sb["throughput_us"], sb["latency_us"]),
                         "hbm_frac_compressed_bytes": round(nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                         "effective_weight_GBs": round(2 * gate.K * gate.N / (us * 1e-6) / 1e9, 1),
                         "mfma_TFLOPs": round(2 * M * gate.K * gate.N / (us * 1e-6) / 1e12, 2),
                         "mfma_util_vs_2500_TFLOPs": round(2 * M * gate.K * gate.N / (us * 1e-6) / 1e12 / 2500.0, 5),
                         "torch_matmul_bf16_us": round(us_ref, 2),
                         "torch_matmul_weight_GBs": round(2 * gate.K * gate.N / (us_ref * 1e-6) / 1e9, 1)})
        out["fused_gemv"] = {"layer": f"gate K={gate.K} N={gate.N}", "bytes_M1": gate.linear_bytes(1), "rows": rows}
        if a.new_kernels:
            # more than 64 rows of x: the fused kernel that decodes once per 64 rows, the one that decodes once per
            # 128 / 256 rows (must give the same bits), and the default policy (decode once to HBM + library GEMM)
            import comp_inference_amd.linear_hip as lh

            wide_rows = []
            for M in GEMM_ROWS:
                xm = torch.randn(M, gate.K, generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev)
                policy = lh.DECODE_ONCE_ABOVE_ROWS
                t_default = batched_time_us(lambda: gate.linear(xm), 5, 20)
                lh.DECODE_ONCE_ABOVE_ROWS = None
                try:
                    lh.fused_wide_rows(False)
                    narrow = gate.linear(xm)
                    t_narrow = batched_time_us(lambda: gate.linear(xm), 5, 20)
                    lh.fused_wide_rows(True)
                    wide = gate.linear(xm)
                    t_wide = batched_time_us(lambda: gate.linear(xm), 5, 20)
                finally:
                    lh.fused_wide_rows(False)
                    lh.DECODE_ONCE_ABOVE_ROWS = policy
                t_ref = batched_time_us(lambda: torch.matmul(xm, w_dense), 5, 20)
                flops = 2.0 * M * gate.K * gate.N
                wide_rows.append({"M": M, "us_one_decode_per_64_rows": round(t_narrow, 1),
                                  "us_one_decode_per_pass": round(t_wide, 1), "bit_identical": bool(torch.equal(narrow, wide)),
                                  "us_decode_once_plus_library_gemm": round(t_default, 1),
                                  "mfma_util_vs_2500_TFLOPs": round(flops / (t_wide * 1e-6) / 1e12 / 2500.0, 4),
                                  "torch_matmul_bf16_us": round(t_ref, 1)})
            out["fused_gemm_rows"] = {"layer": f"gate K={gate.K} N={gate.N}", "rows": wide_rows}

    # --- the four GEMVs of a decoder layer at M = 1 (q/k/v and gate/up fused along the outputs, as the
    # runtime modules hold them), with decoder checkpoints where the library suggests them
    if not a.no_gemv:
        by = {n: w for n, w in make_layer(1)}
        shapes = [("qkv", torch.cat((by["q"], by["k"], by["v"]), 0)), ("o", by["o"]),
                  ("gate_up", torch.cat((by["gate"], by["up"]), 0)), ("down", by["down"])]
        g = torch.Generator("cpu").manual_seed(2)
        rows, total, total_ref = [], 0.0, 0.0
        for name, w in shapes:
            c = Compressed(name, w, dev)
            x = torch.randn(1, c.K, generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev)
            w_dense = w.t().contiguous().to(dev)
            ok = bool(torch.allclose(c.linear_segmented(x).float(), torch.matmul(x, w_dense).float(), atol=1e-2, rtol=1e-2))
            us = batched_time_us(lambda: c.linear_segmented(x), 25, 100)
            us_plain = batched_time_us(lambda: c.linear(x), 25, 100)
            us_ref = batched_time_us(lambda: torch.matmul(x, w_dense), 25, 100)
            total, total_ref = total + us, total_ref + us_ref
            record("fused linear (checkpoints)", f"{name} K={c.K} N={c.N} M=1", c.linear_bytes(1), us)
            rows.append({"layer": f"{name} K={c.K} N={c.N}", "segments": int(c.segments), "us": round(us, 2),
                         "us_without_checkpoints": round(us_plain, 2), "allclose_1e-2": ok,
                         "checkpoint_bytes": 0 if c.checkpoints is None else int(c.checkpoints.numel() * 8),
                         "compressed_bytes": int(c.linear_bytes(1)),
                         "effective_weight_GBs": round(2 * c.K * c.N / (us * 1e-6) / 1e9, 1),
                         "torch_matmul_bf16_us": round(us_ref, 2)})
            del c, w_dense
        out["fused_gemv_layer_M1"] = {"rows": rows, "sum_us": round(total, 1), "sum_torch_matmul_bf16_us": round(total_ref, 1)}

    # --- fused decompress-gather on a 128256 x 4096 table, 2048 Zipf(1.1) ids
    if not a.no_embedding:
        log("generating and compressing the embedding table (seed 3) ...")
        V, H, T = EMBED_SHAPE
        g = torch.Generator("cpu").manual_seed(3)
        table = (torch.randn(V, H, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16)
        emb = Compressed("embed", table, dev, transpose=False)
        p = np.arange(1, V + 1, dtype=np.float64) ** -1.1
        ids_np = np.random.default_rng(4).choice(V, T, p=p / p.sum())
        ids = torch.from_numpy(ids_np).to(dev)

        emb_segments = 8  # decoder checkpoints every 64 rows, as RansEmbedding keeps them
        ck = ci.build_checkpoints(emb.stream, emb.states, emb.tables, emb.slot_map, (V, H), emb.tile_offsets,
                                  emb.tile_max_lens, emb.th, emb.tw, emb_segments)

        def gather(use_ck=True):
            return ci.fused_rans_embedding(ids, emb.stream, emb.states, emb.tables, emb.slot_map, (V, H),
                                           emb.tile_offsets, emb.tile_max_lens, emb.th, emb.tw, emb.man,
                                           checkpoints=ck if use_ck else None, segments=emb_segments if use_ck else 1)

        want_rows = table[torch.from_numpy(ids_np)].view(torch.int16)
        exact = bool(torch.equal(gather().cpu().view(torch.int16), want_rows)) and \
            bool(torch.equal(gather(False).cpu().view(torch.int16), want_rows))
        us = batched_time_us(gather, 10, 50)
        us_no_ck = batched_time_us(lambda: gather(False), 10, 50)
        table_dev = table.to(dev)
        us_ref = batched_time_us(lambda: table_dev[ids], 10, 50)
        out["fused_embedding"] = {"table": f"{V}x{H} bf16 N(0,0.02) seed 3", "ids": f"{T} Zipf(1.1) seed 4",
                                  "distinct_ids": int(np.unique(ids_np).size), "bit_exact": exact, "us": round(us, 1),
                                  "segments": emb_segments, "checkpoint_bytes": int(ck.numel() * 8),
                                  "us_without_checkpoints": round(us_no_ck, 1),
                                  "rows_per_s": round(T / (us * 1e-6), 1),
                                  "gathered_GBs": round(T * H * 2 / (us * 1e-6) / 1e9, 2),
                                  "compressed_table_bytes": int(emb.stream.numel() + emb.man.numel()),
                                  "torch_index_bf16_us": round(us_ref, 1)}
        # useful bytes of the gather: the rows written and, per distinct (half tile of rows, pair of column
        # tiles) touched, nothing less than the rows themselves in compressed form -- counted as output only
        record("embed_gather32_kernel (+ grouping)", f"{V}x{H} table, {T} Zipf ids, 8 segments", T * H * 2 + T * 8, us)
        if a.new_kernels:
            slot_table = ci.build_slot_table(emb.tables, emb.slot_map)

            def gather16():
                return ci.fused_rans_embedding(ids, emb.stream, emb.states, emb.tables, emb.slot_map, (V, H),
                                               emb.tile_offsets, emb.tile_max_lens, emb.th, emb.tw, emb.man,
                                               checkpoints=ck, segments=emb_segments, slot_table=slot_table)

            exact16 = bool(torch.equal(gather16().cpu().view(torch.int16), want_rows))
            us16 = batched_time_us(gather16, 10, 50)
            out["fused_embedding"]["sixteen_wavefronts"] = {"bit_exact": exact16, "us": round(us16, 1)}
            record("embed_gather32_seg_kernel (+ grouping)", f"{V}x{H} table, {T} Zipf ids, 8 segments", T * H * 2 + T * 8, us16)

        # --- the same table as a tied LM head: logits = x W^T, M = 1
        xh = torch.randn(1, H, generator=torch.Generator("cpu").manual_seed(2), dtype=torch.float32).to(torch.bfloat16).to(dev)

        def head():
            return ci.fused_rans_linear_transposed(xh, emb.stream, emb.states, emb.tables, emb.slot_map, (V, H),
                                                   emb.tile_offsets, emb.tile_max_lens, emb.th, emb.tw, emb.man)

        want_logits = torch.matmul(xh, table_dev.t()).float()
        ok = bool(torch.allclose(head().float(), want_logits, atol=1e-2, rtol=1e-2))
        us_h = batched_time_us(head, 5, 20)
        us_h_ref = batched_time_us(lambda: torch.matmul(xh, table_dev.t()), 5, 20)
        head_bytes = emb.stream.numel() + emb.man.numel() + 4 * emb.n_streams + 8 * emb.n_tiles + 5120 + 2 * H + 2 * V
        out["lm_head"] = {"weight": f"{V}x{H} (the embedding table, tied)", "M": 1, "us": round(us_h, 1), "allclose_1e-2": ok,
                          "hbm_frac_compressed_bytes": round(record("trans32_kernel (+ reduction)", f"{V}x{H} head M=1", head_bytes, us_h), 4),
                          "effective_weight_GBs": round(2 * V * H / (us_h * 1e-6) / 1e9, 1),
                          "torch_matmul_bf16_us": round(us_h_ref, 1)}
        if a.new_kernels:
            # the head's sixteen-wavefront kernel for one row of x (decoder checkpoints, largest window from the library),
            # with the sums by lane exchanges (bit-identical to the default) and on the matrix pipe (within tolerance)
            import ctypes as C

            from comp_inference_amd import _lib

            variants = []
            for segs in (2, 4):
                ck_h = ci.build_checkpoints(emb.stream, emb.states, emb.tables, emb.slot_map, (V, H), emb.tile_offsets,
                                            emb.tile_max_lens, emb.th, emb.tw, segs)
                rows_t = torch.zeros(1, dtype=torch.int32, device=dev)
                desc = _lib.tiled_weight(V, H, emb.th, emb.tw, emb.stream, emb.states, emb.tables, emb.slot_map,
                                         emb.tile_offsets, emb.tile_max_lens, None, ck_h, segs)
                _lib.check(_lib.lib().ci_max_window_rows(C.byref(desc), _lib.ptr(rows_t), _lib.stream_handle(dev)))
                kw = dict(checkpoints=ck_h, segments=segs, max_window_rows=int(rows_t.item()),
                          slot_table=ci.build_slot_table(emb.tables, emb.slot_map))

                def head_seg():
                    return ci.fused_rans_linear_transposed(xh, emb.stream, emb.states, emb.tables, emb.slot_map, (V, H),
                                                           emb.tile_offsets, emb.tile_max_lens, emb.th, emb.tw, emb.man, **kw)

                same = bool(torch.equal(head_seg(), head()))
                us_seg = batched_time_us(head_seg, 5, 20)
                ci.head_matrix_sums(True)
                try:
                    close = bool(torch.allclose(head_seg().float(), want_logits, atol=1e-2, rtol=1e-2))
                    us_mat = batched_time_us(head_seg, 5, 20)
                finally:
                    ci.head_matrix_sums(False)
                variants.append({"segments": segs, "max_window_rows": kw["max_window_rows"], "us_lane_exchange_sums": round(us_seg, 1),
                                 "bit_identical_to_default": same, "us_matrix_pipe_sums": round(us_mat, 1), "allclose_1e-2": close})
                del ck_h
            out["lm_head"]["sixteen_wavefronts"] = variants
        del emb, table_dev, table, ck

    roofline["kernels"] = kernels
    if not a.no_cpu_baseline:
        log("timing the CPU oracle ...")
        out["cpu_baseline"] = cpu_baseline(layer)
        out["cpu_roundtrip"] = cpu_roundtrip()
    del layer, items, plain_items
    torch.cuda.empty_cache()

    # --- the whole decoder: 32 layers, 128-token prompt, 256 greedy tokens, weights from the CPU generator
    if not a.no_model:
        import bench_model

        m = bench_model.run(32, 128, 256, 1024, 32, "cpu")
        out["fused_model"] = {k: m[k] for k in (
            "model", "prompt_tokens", "new_tokens", "weight_bytes_compressed", "weight_bytes_bf16",
            "checkpoint_index_bytes", "tok_per_s_compressed_graph", "tok_per_s_compressed_eager",
            "tok_per_s_reference_bf16_graph", "tok_per_s_reference_bf16_eager",
            "ids_equal_to_decompressed_same_order_run", "graph_ids_equal_to_decompressed_same_order_run",
            "teacher_forced_logits_bit_identical_to_same_order_run", "ids_equal_to_reference",
            "teacher_forced_top1_agreement", "teacher_forced_max_abs_logit_diff",
            "reference_smallest_top1_top2_logit_gap")}

    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
