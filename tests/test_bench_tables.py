"""bench.py's recorded counter traffic equals the committed counter summaries it is taken from. CPU only."""
import importlib.util
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def load_bench():
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(ROOT, "bench.py"))
    m = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(m)
    return m


def test_measured_traffic_equals_the_total_line_of_its_counter_summary():
    bench = load_bench()
    assert set(bench.MEASURED_TRAFFIC_BYTES) == set(bench.TRAFFIC_PROFILES)
    for key, stem in bench.TRAFFIC_PROFILES.items():
        text = open(os.path.join(ROOT, "profiles", stem + "_hbm_traffic.txt")).read()
        assert "--workload %s " % key in text or (key == "fused" and "bench.py --workload fused " in text), key
        read = int(re.search(r"^\s*read\s+(\d+) bytes", text, re.M).group(1))
        write = int(re.search(r"^\s*write\s+(\d+) bytes", text, re.M).group(1))
        total = int(re.search(r"^\s*total\s+(\d+) bytes", text, re.M).group(1))
        assert read + write == total, key
        assert bench.MEASURED_TRAFFIC_BYTES[key] == total, key


def test_every_workload_named_in_a_profile_exists():
    bench = load_bench()
    for f in sorted(os.listdir(os.path.join(ROOT, "profiles"))):
        for wl in re.findall(r"bench\.py --workload (\S+)", open(os.path.join(ROOT, "profiles", f)).read()):
            assert wl in bench.WORKLOADS, (f, wl)
