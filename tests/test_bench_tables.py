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


def test_byte_conventions_of_the_baseline_configurations():
    """The three byte counts a launch can be priced with, from the operators' own index maps: the row spans
    (`roofline.achieved`), whole tensors, referenced pixels only. The expected numbers are closed forms of the
    configurations' shapes (448 distinct rows and columns for 224 bilinear outputs, 4 taps per output for bicubic)."""
    b = load_bench()
    rows, span = b.span_bytes(224, 16, 1080, 256, b.LINEAR, 1)[0], b.span_bytes(224, 115, 1920, 455, b.LINEAR, 3)[1]
    cols = b.span_bytes(224, 115, 1920, 455, b.LINEAR, 3)[0]
    out = 3 * 224 * 224 * 4
    assert (rows, cols, span) == (448, 448, 2829)
    assert (rows * span + out) * 64 == 119648256            # fused, row spans
    assert (rows * cols * 3 + out) * 64 == 77070336          # referenced pixels only
    assert (1080 * 1920 * 3 + out) * 64 == 436666368         # whole tensors
    rows, cols = b.span_bytes(224, 0, 1080, 224, b.LINEAR, 1)[0], b.span_bytes(224, 0, 1920, 224, b.LINEAR, 3)[0]
    assert (rows * cols + 224 * 224) * 3 * 8 == 6021120      # Resize LINEAR 1080p -> 224, batch 8
    rows, cols = b.span_bytes(224, 0, 1080, 224, b.NEAREST, 1)[0], b.span_bytes(224, 0, 1920, 224, b.NEAREST, 3)[0]
    assert (rows, cols) == (224, 224)
    rows, cols = b.span_bytes(360, 0, 2160, 360, b.CUBIC, 1)[0], b.span_bytes(640, 0, 3840, 640, b.CUBIC, 16)[0]
    assert (rows, cols) == (1440, 2560) and (rows * cols + 360 * 640) * 16 * 16 == 1002700800


def test_the_byte_movers_move_at_least_the_bytes_of_the_operators_they_stand_beside():
    """`roofline.dense_mover` compares an operator with a kernel that only moves bytes: the mover's reads and writes
    are each at least the operator's (fused: 448 x 2829 bytes of row spans read and 602112 written per image; NV12:
    1.5 and 3 bytes per pixel; cubic: the row spans and the 640 x 360 x 16-byte output)."""
    b = load_bench()
    specs = b.StreamMix.SPECS

    def moved(key):
        reads, writes, lanes = specs[key]
        return 16 * lanes * reads, 16 * lanes * writes
    assert b.Nv12C3.mover in specs and b.CubicC5.mover in specs
    r, w = moved("stream-mix-4-2")
    assert r >= 64 * 448 * 2829 and w >= 64 * 602112 and r + w <= 1.02 * 119648256
    r, w = moved(b.Nv12C3.mover)
    assert (r, w) == (32 * 1620 * 1920, 32 * 1080 * 1920 * 3)
    r, w = moved(b.CubicC5.mover)
    assert w == 16 * 640 * 360 * 16 and r >= 1473822720 - w and r + w <= 1.001 * 1473822720
