"""The counter arithmetic of bench.py's --traffic-summary and --counter-summary on a synthetic counter file (no GPU)."""
import csv
import json
import os
import subprocess
import sys

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def write_counter_file(path, counter, per_launch_units):
    """A rocprofv3 --pmc CSV as bench.py --traffic-probe would leave it: per workload two untimed launches, a marker,
    the counted launches, a marker; one other kernel outside the markers."""
    rows, did = [], 0

    def add(kernel, value):
        nonlocal did
        did += 1
        rows.append({"Dispatch_Id": did, "Kernel_Name": kernel, "Counter_Name": counter, "Counter_Value": value})

    for units in per_launch_units:
        add("warm_up_kernel", 12345)
        add("warm_up_kernel", 12345)
        add(f"void sa::{bench.MARKER_KERNEL}(Params)", 1)
        for i in range(bench.TRAFFIC_PROBE_LAUNCHES):
            add("work_kernel_a", units * 0.75)
            add("work_kernel_b", units * 0.25)
        add(f"void sa::{bench.MARKER_KERNEL}(Params)", 1)
    with open(path, "w", newline="") as fh:
        w = csv.DictWriter(fh, fieldnames=list(rows[0]))
        w.writeheader()
        w.writerows(reversed(rows))  # the summaries sort by dispatch id themselves


def run(*args):
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    return json.loads(r.stdout)


def test_traffic_summary_scales_by_the_copy(tmp_path):
    n = len(bench.PROBE_WORKLOADS)
    assert bench.PROBE_WORKLOADS[-1] == "copy 1 GiB"
    fetch_units = [1000.0 * (i + 1) for i in range(n - 1)] + [524288.0]   # the copy reads 2^30 bytes: 2048 per unit
    write_units = [10.0 * (i + 1) for i in range(n - 1)] + [1048576.0]    # and writes 2^30 bytes: 1024 per unit
    f, w = str(tmp_path / "f.csv"), str(tmp_path / "w.csv")
    write_counter_file(f, "FETCH_SIZE", fetch_units)
    write_counter_file(w, "WRITE_SIZE", write_units)
    out = run("--traffic-summary", f, w)
    assert out["bytes_per_FETCH_SIZE_unit"] == 2048.0 and out["bytes_per_WRITE_SIZE_unit"] == 1024.0
    for i, name in enumerate(bench.PROBE_WORKLOADS[:-1]):
        assert out["workloads"][name] == [round(fetch_units[i] * 2048), round(write_units[i] * 1024)]
    assert out["workloads"]["copy 1 GiB"] == [1 << 30, 1 << 30]
    assert set(bench.TRAFFIC_BYTES) == set(bench.PROBE_WORKLOADS[:-1])  # every probed workload has its constants


def test_counter_summary_is_per_launch(tmp_path):
    n = len(bench.PROBE_WORKLOADS)
    units = [7.0 * (i + 1) for i in range(n)]
    path = str(tmp_path / "s.csv")
    write_counter_file(path, "SQ_INSTS_MFMA", units)
    out = run("--counter-summary", path)
    for i, name in enumerate(bench.PROBE_WORKLOADS):
        assert abs(out[name]["SQ_INSTS_MFMA"] - units[i]) < 1e-9


def test_a_file_with_a_missing_span_is_refused(tmp_path):
    path = str(tmp_path / "s.csv")
    write_counter_file(path, "SQ_INSTS_MFMA", [1.0, 2.0])
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--counter-summary", path], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "marked spans" in (r.stderr + r.stdout)


def test_traffic_digests_name_the_sources_in_the_tree():
    # the traffic constants were read with the kernels that are in the tree (a kernel edit must re-run the probe)
    for which, digest in bench.TRAFFIC_KERNEL_SOURCES_SHA16.items():
        assert bench.kernel_sources_sha16(which) == digest, which
