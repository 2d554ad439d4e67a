"""Builds the two shared libraries of this package with hipcc for gfx950:

  lib/libnvcv_types.so  -- NVCV core objects (host C++ on the HIP runtime)
  lib/libcvcuda.so      -- operators: host validation/dispatch + HIP kernels
  lib/libcvamd_bench.so -- kernels the benchmark times beside the operators (a copy-bound twin of the
                           fused kernel); nothing in the two libraries above uses it

Usage: python cv-cuda_amd/build.py [--force] [-j N]
Objects are cached under build/ next to this file and rebuilt when a source or header is newer.
"""
import argparse
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(ROOT, "include")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "build")
ARCH = "gfx950"

COMMON = [
    "-std=c++17", "-O3", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wextra", "-Wno-unused-parameter",
    "-I" + INCLUDE, "-I" + CSRC,
]
# Device code: no FMA contraction (results must match the CPU goldens' expression shapes), no
# packed-FP32 instruction selection, and no v_ashr_pk_{u8,i8}_i32: the compiler treats the upper 16 bits
# of that instruction's result as zero, on MI355X they held the destination's previous contents (seen
# as wrong third bytes where two clamped shifts were OR-ed with a third in the 4:2:0 -> RGB kernel).
DEVICE = [
    "--offload-arch=" + ARCH, "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Xclang", "-target-feature", "-Xclang", "-ashr-pk-insts",
]


def _sources(sub, exts):
    d = os.path.join(CSRC, sub)
    return sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith(exts))


def _headers():
    out = []
    for base in (INCLUDE, CSRC):
        for dp, _, fs in os.walk(base):
            out += [os.path.join(dp, f) for f in fs if f.endswith((".h", ".hpp", ".inc"))]
    return out


def _compile(src, obj, extra, force, newest_header):
    if (not force and os.path.exists(obj) and os.path.getmtime(obj) >= os.path.getmtime(src)
            and os.path.getmtime(obj) >= newest_header):
        return None
    cmd = ["hipcc"] + COMMON + extra + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    msgs = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                     if ("packed-fp32-ops" not in l and "ashr-pk-insts" not in l) or "error" in l)
    if r.returncode != 0:
        raise RuntimeError("compile failed: %s\n%s" % (" ".join(cmd), msgs))
    return msgs


def build(force=False, jobs=8, verbose=True):
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    newest_header = max(os.path.getmtime(h) for h in _headers())
    core = [(s, []) for s in _sources("nvcv", (".cpp",))]
    ops = [(s, DEVICE if s.endswith(".hip") else []) for s in _sources("cvcuda", (".cpp", ".hip"))]
    bench = [(s, DEVICE) for s in _sources("bench", (".hip",))]
    tasks = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        for group, items in (("nvcv", core), ("cvcuda", ops), ("bench", bench)):
            for src, extra in items:
                obj = os.path.join(OBJDIR, group + "_" + os.path.basename(src) + ".o")
                tasks.append((group, obj, ex.submit(_compile, src, obj, extra, force, newest_header)))
        for group, obj, fut in tasks:
            msgs = fut.result()
            if verbose and msgs:
                print(msgs)
    core_objs = [o for g, o, _ in tasks if g == "nvcv"]
    ops_objs = [o for g, o, _ in tasks if g == "cvcuda"]
    nvcv_so = os.path.join(LIBDIR, "libnvcv_types.so")
    cvcuda_so = os.path.join(LIBDIR, "libcvcuda.so")
    link = ["hipcc", "-shared", "-fPIC", "--offload-arch=" + ARCH, "-Wl,--no-undefined"]
    # ELF symbol versions of the reference's ABI (FUNC@@NVCV_x.y / FUNC@@CVCUDA_x.y), see csrc/abi
    maps = os.path.join(CSRC, "abi")
    subprocess.run(link + core_objs + ["-o", nvcv_so, "-Wl,-soname,libnvcv_types.so",
                                       "-Wl,--version-script=" + os.path.join(maps, "nvcv_types.map")], check=True)
    subprocess.run(link + ops_objs + ["-o", cvcuda_so, "-Wl,-soname,libcvcuda.so", "-L" + LIBDIR, "-lnvcv_types",
                                      "-Wl,-rpath,$ORIGIN",
                                      "-Wl,--version-script=" + os.path.join(maps, "cvcuda.map")], check=True)
    bench_so = os.path.join(LIBDIR, "libcvamd_bench.so")
    subprocess.run(link + [o for g, o, _ in tasks if g == "bench"] + ["-o", bench_so], check=True)
    return nvcv_so, cvcuda_so, bench_so


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("-j", type=int, default=8)
    a = ap.parse_args()
    print("\n".join(build(a.force, a.j)))
