"""bench.py reports roofline.traffic only while the kernel sources are the ones the counters were read on."""
import importlib.util
import json
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


HEADER = ('"Correlation_Id","Dispatch_Id","Agent_Id","Queue_Id","Process_Id","Thread_Id","Grid_Size","Kernel_Id","Kernel_Name",'
          '"Workgroup_Size","LDS_Block_Size","Scratch_Size","VGPR_Count","Accum_VGPR_Count","SGPR_Count","Counter_Name",'
          '"Counter_Value","Start_Timestamp","End_Timestamp"\n')


def _csv(path, counter, rows):
    with open(path, "w") as f:
        f.write(HEADER)
        for i, (kernel, value) in enumerate(rows, 1):
            f.write(f'{i},{i},"Agent 1",1,1,1,64,7,"{kernel}",64,0,0,8,0,16,"{counter}",{value:.6f},1,2\n')


def test_counter_files_become_a_record_tied_to_the_sources(tmp_path, monkeypatch):
    b = _bench()
    monkeypatch.setattr(b, "TRAFFIC_JSON", str(tmp_path / "traffic.json"))
    seg = "void ci::decode_tiled32_seg_kernel<false>(ci::DecodeBatchArgs)"
    copy = "__amd_rocclr_copyBuffer"
    # three calibration copies of 64 MiB first (the fetch counter reads half of the bytes on this chip), later copies of
    # other sizes are uploads and do not count
    _csv(tmp_path / "f.csv", "FETCH_SIZE", [(copy, 32768.0)] * 3 + [(copy, 11.0), (seg, 70000.0), (seg, 72000.0)])
    _csv(tmp_path / "w.csv", "WRITE_SIZE", [(copy, 65536.0)] * 3 + [(copy, 5.0), (seg, 200000.0), (seg, 200000.0)])
    assert b.record_traffic(str(tmp_path / "f.csv"), str(tmp_path / "w.csv")) == 0
    rec = json.load(open(tmp_path / "traffic.json"))
    assert rec["fetch_scale"] == 2.0 and rec["write_scale"] == 1.0
    assert rec["bytes"] == int((71000.0 * 2.0 + 200000.0) * 1024) and rec["sources"] == b.sources_digest()
    assert b.measured_traffic()[0] == rec["bytes"]
    # a change to any kernel source: the figure is no longer reported
    rec["sources"] = "0" * 16
    json.dump(rec, open(tmp_path / "traffic.json", "w"))
    got, why = b.measured_traffic()
    assert got is None and "not carried over" in why
    os.remove(tmp_path / "traffic.json")
    assert b.measured_traffic()[0] is None


def test_the_committed_record_is_well_formed():
    rec = json.load(open(os.path.join(ROOT, "profiles", "traffic.json")))
    assert rec["kernel"] == "decode_tiled32_seg_kernel" and isinstance(rec["bytes"], int) and len(rec["sources"]) == 16
    assert abs(rec["bytes"] - (rec["fetch_kib"] * rec["fetch_scale"] + rec["write_kib"] * rec["write_scale"]) * 1024) < 4096
