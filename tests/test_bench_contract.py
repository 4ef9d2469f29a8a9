"""bench.py's host-side pieces, without a GPU: the configuration list, the buffer-set rule, the traffic table it reads
from profiles/, and the refusal of more than one GPU."""
import importlib.util
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def load_bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_configuration_names_select_one_configuration_each():
    bench = load_bench()
    names = bench.CONFIG_NAMES
    assert bench.HEADLINE in names and len(set(names)) == len(names)
    for n in names:
        assert [m for m in names if m.startswith(n)] == [n]


def test_buffer_sets_move_more_than_the_cache_between_two_uses():
    bench = load_bench()
    for nbytes in (20e6, 37e6, 136e6, 199e6, 404e6):
        sets = bench.sets_for(nbytes)
        assert sets * nbytes >= 1.5 * bench.CACHE_BYTES and sets <= bench.MAX_SETS
    assert bench.sets_for(1.4e9) == 1  # a launch that moves five times the cache needs no second set
    small = bench.Workload("tiny", None, 1, 234096, "k", bench.sets_for(234096), None)
    assert small.cache_resident and "frac_peak_cache_resident" in small.roofline(0.005) and "frac" not in small.roofline(0.005)


def test_traffic_comes_from_the_profile_summary():
    bench = load_bench()
    traffic, source = bench.measured_traffic(bench.HEADLINE)
    assert traffic is not None and "profiles/hbm_traffic.md" in source and "commit" in source
    head = bench.Workload(bench.HEADLINE, None, 10368000, 136212480, "k", 4, None)
    r = head.roofline(0.0244)
    assert r["bound"] == "hbm" and r["peak"] == 8000.0 and abs(r["frac"] - 136212480 / 0.0244e-3 / 8e12) < 1e-12
    assert 0.95 * r["alg_bytes_per_launch"] < r["traffic"] < 1.3 * r["alg_bytes_per_launch"]
    assert bench.measured_traffic("no_such_configuration") == (None, None)


def test_more_than_one_gpu_is_refused_with_a_message():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert out.returncode != 0 and "one GPU" in out.stderr
