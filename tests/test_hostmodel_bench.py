"""bench.py from its first line to its JSON line, on the host model (tests/hostmodel): the same code path the GPU
run takes -- compression, the bit-exact checks before every timed region, every workload of the line including the
ones behind --new-kernels, the CPU baseline, the decoder loop -- with the workloads' shapes made small and each timing loop run once
(no time passes on the model, so the figures themselves mean nothing; the keys, the checks and the arithmetic
around them do)."""
import io
import json
import sys
from contextlib import redirect_stdout

from tests.hostmodel.model import in_fresh_process


@in_fresh_process
def test_bench_runs_from_start_to_its_json_line():
    from tests.hostmodel.backend import python_api_on_hostmodel

    with python_api_on_hostmodel(cus=8):
        import bench

        # (name, out, in): in = K >= one tile of 1024 rows; a ragged k tile in `down`
        bench.LAYER = [("q", 64, 1024), ("k", 32, 1024), ("v", 32, 1024), ("o", 64, 1024),
                       ("gate", 96, 2048), ("up", 96, 2048), ("down", 64, 1300)]
        bench.GEMV_ROWS = (1, 4, 16)
        bench.GEMM_ROWS = (16, 130)
        bench.EMBED_SHAPE = (2048 + 256, 64, 48)
        bench.batched_time_us = lambda fn, warmup, iters: (fn(), 10.0)[1]
        bench.event_times_us = lambda fn, warmup, iters: (fn(), [10.0])[1]
        # the decoder of the last section: two layers of a narrow model, eight prompt tokens, six new ones, tiles of
        # 64 rows; every generation eager (a HIP graph is the GPU runtime's to capture)
        import bench_model

        for name, v in dict(hidden=128, ffn=256, heads=4, kv_heads=2, head_dim=32, vocab=512).items():
            setattr(bench_model.Shape, name, v)
        bench_model.generate = lambda dec, prompt, n_new, use_graph, _g=bench_model.generate: _g(dec, prompt, n_new, False)
        bench_model.run = lambda *a, _r=bench_model.run: _r(2, 8, 6, 64, 32, "cpu")
        argv, sys.argv = sys.argv, ["bench.py", "--steps", "2", "--warmup", "1", "--new-kernels"]
        buf = io.StringIO()
        try:
            with redirect_stdout(buf):
                assert bench.main() == 0
        finally:
            sys.argv = argv
    lines = [ln for ln in buf.getvalue().splitlines() if ln.strip()]
    assert len(lines) == 1, lines  # ONE JSON line on stdout
    out = json.loads(lines[0])
    for key, kind in (("metric", str), ("value", float), ("unit", str), ("n_gpus", int), ("steps", int), ("warmup", int),
                      ("ms_per_step", float), ("higher_is_better", bool), ("scaling", str), ("dtype", str), ("data", str),
                      ("config", dict), ("roofline", dict), ("cpu_baseline", dict)):
        assert isinstance(out[key], kind), (key, out[key])
    assert out["n_gpus"] == 1 and out["steps"] == 2 and out["warmup"] == 1 and out["vs_baseline"] is None
    assert out["dtype"] == "u8" and "workload" in out["config"] and "model" not in out["config"]
    r = out["roofline"]
    assert r["bound"] == "hbm" and r["unit"] == "GB/s" and r["peak"] == 8000.0 and "traffic" in r
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3
    assert {k["kernel"] for k in r["kernels"]} >= {"decode_tiled32_seg_kernel", "fused linear (checkpoints)",
                                                   "embed_gather32_seg_kernel (+ grouping)", "trans32_kernel (+ reduction)"}
    c = out["cpu_baseline"]
    assert c["kind"] == "port" and c["cores"] >= 1 and c["unit"] == "GB/s" and c["value"] > 0 and c["sample"]
    assert out["cpu_roundtrip"]["bit_exact"] is True
    m = out["fused_model"]
    assert m["ids_equal_to_decompressed_same_order_run"] and m["teacher_forced_logits_bit_identical_to_same_order_run"]
    assert m["new_tokens"] == 6 and m["weight_bytes_compressed"] < m["weight_bytes_bf16"]
    # every check the bench makes of what it times came out right
    assert all(row["allclose_1e-2"] for row in out["fused_gemv"]["rows"])
    assert all(row["allclose_1e-2"] for row in out["fused_gemv_layer_M1"]["rows"])
    assert all(row["bit_identical"] for row in out["fused_gemm_rows"]["rows"])
    assert out["fused_embedding"]["bit_exact"] and out["fused_embedding"]["sixteen_wavefronts"]["bit_exact"]
    assert out["lm_head"]["allclose_1e-2"]
    assert all(v["bit_identical_to_default"] and v["allclose_1e-2"] for v in out["lm_head"]["sixteen_wavefronts"])
