"""bench.py --traffic-from: the record the roofline's `traffic` figure is read
from is rebuilt from rocprofv3 counter CSVs (synthetic ones here), scaled by
the calibration copy, stamped with the kernel-source digest, and refused by
the reader when the sources have changed since."""
import csv
import importlib.util
import json
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", ROOT / "bench.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _write_run(directory, counter, rows):
    directory.mkdir(parents=True)
    with open(directory / "pmc_counter_collection.csv", "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=["Kernel_Name", "Counter_Name", "Counter_Value"])
        w.writeheader()
        for name, value in rows:
            w.writerow({"Kernel_Name": name, "Counter_Name": counter, "Counter_Value": value})


def test_traffic_record_round_trip(tmp_path, monkeypatch):
    bench = _bench()
    kib = 1 << 20  # the calibration copy moves 2^20 KiB each way
    for workload, kernel in bench.DOMINANT_KERNEL.items():
        # FETCH_SIZE counts in double units on this part (the copy reads half), WRITE_SIZE exactly
        _write_run(tmp_path / f"pmc_FETCH_SIZE_{workload}", "FETCH_SIZE",
                   [(f"void ic::{kernel}<a, b>(args)", 1000.0), (f"void ic::{kernel}<a, b>(args)", 1002.0),
                    ("__amd_rocclr_copyBuffer", kib / 2 + 10.0), ("__amd_rocclr_copyBuffer", 3.0),
                    ("void at::native::elementwise_copy_kernel", 700000.0), ("kv_append_kernel", 5.0)])
        _write_run(tmp_path / f"pmc_WRITE_SIZE_{workload}", "WRITE_SIZE",
                   [(f"void ic::{kernel}<a, b>(args)", 10.0), ("__amd_rocclr_copyBuffer", float(kib))])
    out = tmp_path / "traffic.json"
    monkeypatch.setattr(bench, "TRAFFIC_FILE", str(out))
    rec = bench.traffic_record(str(tmp_path), seed=0)
    assert sorted(rec["workloads"]) == sorted(bench.DOMINANT_KERNEL)
    ent = json.loads(out.read_text())["workloads"]["prefill"]
    assert ent["FETCH_SIZE"] == 1001.0 and abs(ent["FETCH_SIZE_scale"] - 2.0) < 1e-3
    assert ent["WRITE_SIZE_scale"] == 1.0
    assert abs(ent["hbm_bytes_per_launch"] - (1001.0 * 2.0 + 10.0) * 1024) < 64
    # the reader hands the figure out for the sources it was measured on, and only for them
    got, stale = bench.measured_traffic("prefill", 0)
    assert got == ent["hbm_bytes_per_launch"] and not stale
    assert bench.measured_traffic("prefill", 1) == (None, False)       # another seed: another workload
    data = json.loads(out.read_text())
    data["csrc_sha256"] = "0" * 64
    out.write_text(json.dumps(data))
    assert bench.measured_traffic("prefill", 0) == (None, True)


def test_traffic_record_skips_workloads_without_runs(tmp_path, monkeypatch):
    bench = _bench()
    monkeypatch.setattr(bench, "TRAFFIC_FILE", str(tmp_path / "traffic.json"))
    rec = bench.traffic_record(str(tmp_path), seed=0)
    assert rec["workloads"] == {}
