"""CPU-only checks of bench.py's host-side pieces: the one-GPU rule, the PMC traffic summary and the JSON that the
bench line's roofline.traffic is read from.  Nothing here touches a GPU."""

import csv
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, BENCH, "--gpus", "2"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert proc.returncode == 2
    assert "ONE GPU" in proc.stderr and proc.stdout.strip() == ""


def _write_counter_csv(directory, counter, per_kernel):
    os.makedirs(os.path.join(directory, "host", "1"), exist_ok=True)
    with open(os.path.join(directory, "host", "1", "p_counter_collection.csv"), "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(["Correlation_Id", "Dispatch_Id", "Kernel_Name", "Counter_Name", "Counter_Value"])
        i = 0
        for name, values in per_kernel.items():
            for v in values:
                i += 1
                w.writerow([i, i, name, counter, v])
                w.writerow([i, i, name, "SOME_OTHER_COUNTER", 1.0])  # rows of other counters are ignored


def test_traffic_summary_scales_by_the_copy_kernel(tmp_path, monkeypatch):
    """Synthetic rocprofv3 CSVs: FETCH_SIZE reads half of the true bytes (as on this part), WRITE_SIZE all of them;
    the 256 MiB copy calibrates both and the kernels' means are scaled accordingly."""
    sys.path.insert(0, ROOT)
    import bench

    ns = "void segpt::(anonymous namespace)::"
    fetch = {"__amd_rocclr_copyBuffer": [10.0, 131072.0, 20.0],  # small uploads and the 256 MiB calibration copy
             ns + "kv_prep_kernel<64>(segpt::KArgs)": [6000.0, 6200.0],
             ns + "fwd_bf16_kernel<64, false, false>(segpt::KArgs)": [40000.0, 40000.0],
             ns + "bwd_dq_bf16_kernel<64, false>(segpt::KArgs)": [90000.0],
             ns + "bwd_dkdv_bf16_kernel<64, false>(segpt::KArgs)": [88000.0, 90000.0]}
    write = {"__amd_rocclr_copyBuffer": [262144.0],
             ns + "kv_prep_kernel<64>(segpt::KArgs)": [12288.0],
             ns + "fwd_bf16_kernel<64, false, false>(segpt::KArgs)": [38016.0],
             ns + "bwd_dq_bf16_kernel<64, false>(segpt::KArgs)": [76608.0],
             ns + "bwd_dkdv_bf16_kernel<64, false>(segpt::KArgs)": [24576.0]}
    fd, wd = str(tmp_path / "f"), str(tmp_path / "w")
    _write_counter_csv(fd, "FETCH_SIZE", fetch)
    _write_counter_csv(wd, "WRITE_SIZE", write)
    out = str(tmp_path / "traffic.json")
    monkeypatch.setattr(bench, "TRAFFIC_JSON", out)
    bench.traffic_from_pmc(fd, wd, 256)
    d = json.load(open(out))
    assert d["FETCH_SIZE_factor"] == 2.0 and d["WRITE_SIZE_factor"] == 1.0
    k = d["kernels"]["bwd_dkdv_bf16_kernel"]
    assert abs(k["read_mb"] - 89000.0 * 1024 * 2 / 1e6) < 0.06 and abs(k["write_mb"] - 24576.0 * 1024 / 1e6) < 0.06
    assert set(d["kernels"]) == {"kv_prep_kernel", "fwd_bf16_kernel", "bwd_dq_bf16_kernel", "bwd_dkdv_bf16_kernel"}
    # what the bench line reports for the dominant kernel: read + write, in bytes
    assert bench.pmc_traffic_bytes("bwd_dkdv") == round((k["read_mb"] + k["write_mb"]) * 1e6)
    monkeypatch.setattr(bench, "TRAFFIC_JSON", str(tmp_path / "absent.json"))
    assert bench.pmc_traffic_bytes("bwd_dkdv") is None


def test_committed_traffic_profile_is_readable():
    sys.path.insert(0, ROOT)
    import bench

    d = json.load(open(bench.TRAFFIC_JSON))
    assert d["copy_mib"] > 0 and 1.5 < d["FETCH_SIZE_factor"] < 2.5 and 0.9 < d["WRITE_SIZE_factor"] < 1.1
    for stage in ("fwd", "bwd_dq", "bwd_dkdv"):
        b = bench.pmc_traffic_bytes(stage)
        assert b is not None and 50e6 < b < 500e6, (stage, b)
