"""bench.py's reported figures are tied to the tracked profile summaries (CPU only)."""

import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_measured_traffic_is_read_from_the_tracked_profiles():
    """`roofline.traffic` of the bench line is the number a profile summary records for that
    workload, preset and kernel -- for the headline workload there must be one, and it must be the
    sum of the scaled FETCH_SIZE and WRITE_SIZE figures of the same file."""
    import bench
    got = bench.measured_traffic("c3", "mi355x", "stage1", "fp16")
    assert got is not None and 1e8 < got < 3e8
    text = open(os.path.join(ROOT, "profiles", "stage1_c3_fp16.txt")).read()
    m = re.search(r"stage1_fused_kernel<F16, 128, false>\(Stage1Args\)\s+read\s+(\d+) KiB.*?write\s+(\d+) KiB", text)
    assert m and abs((int(m.group(1)) + int(m.group(2))) * 1024 - got) <= 2048
    for wl, dt in (("c1", "fp16"), ("c2", "fp16"), ("c4", "bf16"), ("c5", "fp16")):
        assert bench.measured_traffic(wl, "mi355x", "stage1", dt) is not None, wl
    assert bench.measured_traffic("c3", "reference", "stage1", "fp16") is None    # no such run is on record
    assert bench.measured_traffic("c9", "mi355x", "stage1", "fp16") is None


def test_profiles_name_the_command_that_made_them():
    for name in os.listdir(os.path.join(ROOT, "profiles")):
        text = open(os.path.join(ROOT, "profiles", name)).read()
        profiled = "rocprofv3" in text and ("python3 bench.py" in text or "python3 benchmark.py" in text)
        assert profiled or "python3 run_benchmark.py" in text, name     # (a table the sweep wrote: no profiler)


def test_more_than_one_gpu_is_refused():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert out.returncode == 2 and "ONE GPU" in out.stderr


def test_value_is_the_cold_median_after_a_write_flush():
    """`value` keeps one definition across builds: the median over the cold calls, each timed after
    the flush buffer was rewritten and not read back (the reference's do_bench method,
    kernel_bench/benchmark.py:35,59); the figure after a flush that leaves clean lines is a side
    figure under latency_us."""
    import bench
    assert bench.VALUE_METHOD == "cold_median_after_write_flush"
    text = open(os.path.join(ROOT, "bench.py")).read()
    body = text[text.index("cold, warm = [], []"):text.index("cold_clean = []")]
    assert "flush_caches(clean=False)" in body and "flush_caches(clean=True)" not in body and "flush_caches()" not in body
    assert '"value": cold_med if parity["passed"] else None' in text and '"value_method": VALUE_METHOD' in text
    assert '"cold_clean_median"' in text
