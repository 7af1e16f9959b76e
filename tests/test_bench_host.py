"""Host-side parts of bench.py that need no GPU: the refusal of more than one GPU, the provenance of the traffic
figure, the telemetry sampler on a machine without the sysfs files, and the cost model's constants."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2 and "ONE GPU" in r.stderr and r.stdout == ""


def test_traffic_figure_comes_from_the_tracked_record_with_its_commit():
    rec = json.load(open(bench.GEMM_TRAFFIC_RECORD))
    total, why = bench.gemm_traffic(rec["m_tokens"], rec["scaling"])
    assert total == rec["fetch_bytes_per_launch"] + rec["write_bytes_per_launch"]
    assert rec["commit"] in why and os.path.basename(bench.GEMM_TRAFFIC_RECORD) in why
    # scaled counters: raw KiB x factor x 1024, factor = bytes of the calibration copy / what the counter read for it
    cal = rec["calibration"]
    assert abs(cal["copy_bytes"] / (cal["fetch_size_raw_KiB"] * 1024) - cal["fetch_factor"]) < 1e-3
    assert abs(cal["copy_bytes"] / (cal["write_size_raw_KiB"] * 1024) - cal["write_factor"]) < 1e-3
    assert abs(rec["fetch_size_raw_KiB_per_dispatch"] * cal["fetch_factor"] * 1024 - rec["fetch_bytes_per_launch"]) < 1e6
    assert abs(rec["write_size_raw_KiB_per_dispatch"] * cal["write_factor"] * 1024 - rec["write_bytes_per_launch"]) < 1e6
    # every command of the record runs this script
    assert all("-- python3 bench.py" in c for c in rec["commands"])
    # another workload than the recorded one gets no figure
    assert bench.gemm_traffic(rec["m_tokens"] // 2, rec["scaling"])[0] is None
    assert bench.gemm_traffic(rec["m_tokens"], "delayed")[0] is None


def test_algorithmic_bytes_of_the_record_match_the_shapes():
    rec = json.load(open(bench.GEMM_TRAFFIC_RECORD))
    m = rec["m_tokens"]
    # per GEMM: both fp8 operands once + the bf16 result once; three products per shape
    tot = 0
    for _, k, n in bench.SHAPES:
        tot += (m * k + n * k + 2 * m * n) + (m * n + n * k + 2 * m * k) + (m * n + m * k + 2 * n * k)
    assert abs(tot / 12 - rec["algorithmic_bytes_per_launch"]) / rec["algorithmic_bytes_per_launch"] < 0.01


def test_telemetry_is_silent_where_the_sysfs_files_are_missing(tmp_path, monkeypatch):
    t = bench.Telemetry()
    if t.power_file is None:  # no AMD GPU here: start / stop must be harmless
        t.start()
        assert t.stop() is None
    # with files that look like the driver's, it samples them
    dev = tmp_path / "card0" / "device"
    hw = dev / "hwmon" / "hwmon0"
    hw.mkdir(parents=True)
    (hw / "power1_input").write_text("1234000000\n")
    (hw / "power1_cap").write_text("1400000000\n")
    (dev / "pp_dpm_sclk").write_text("0: 132Mhz\n1: 1903Mhz *\n2: 2400Mhz\n")
    import glob as _glob

    real = _glob.glob
    monkeypatch.setattr(_glob, "glob", lambda pat: real(pat.replace("/sys/class/drm", str(tmp_path))))
    t = bench.Telemetry(period=0.001)
    assert t.power_file is not None and t.cap_w == 1400.0
    t.start()
    import time

    time.sleep(0.02)
    r = t.stop()
    assert r["socket_power_W_mean"] == 1234.0 and r["sclk_MHz_mean"] == 1903.0 and r["samples"] >= 2
