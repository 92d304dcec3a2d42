"""Host-side pieces of bench.py and of the benchmark's yardstick library that need no GPU."""
import ctypes
import importlib.util
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "one GPU" in r.stderr


def test_power_sampler_reads_a_hwmon_file_and_copes_without_one(tmp_path, monkeypatch):
    bench = _bench()
    # a box that shows no power file: nothing is sampled, the mean is None
    import glob as glob_mod

    monkeypatch.setattr(glob_mod, "glob", lambda pattern: [])
    with bench.PowerSampler() as ps:
        time.sleep(0.05)
    assert ps.file is None and ps.cap_w is None and ps.mean(0.0, time.perf_counter()) is None
    # a box that does: microwatts in power1_input, the limit in power1_cap
    d = tmp_path / "hwmon0"
    d.mkdir()
    (d / "power1_input").write_text("1234000000\n")
    (d / "power1_cap").write_text("1400000000\n")
    monkeypatch.setattr(glob_mod, "glob", lambda pattern: [str(d)])
    t0 = time.perf_counter()
    with bench.PowerSampler() as ps:
        time.sleep(0.1)
    assert ps.cap_w == 1400.0
    assert len(ps.samples) >= 2
    assert ps.mean(t0, time.perf_counter()) == 1234.0
    assert ps.mean(t0 - 10.0, t0 - 5.0) is None


def test_yardstick_library_exports_its_entry_points():
    lib = ctypes.CDLL(os.path.join(ROOT, "aici_amd", "libmembench.so"))
    for name in ("membench_probe", "membench_mfma_stream"):
        assert hasattr(lib, name)
