"""Builds the two shared libraries of this package with hipcc for gfx950:

  lib/libnvcv_types.so  -- NVCV core objects (host C++ on the HIP runtime)
  lib/libcvcuda.so      -- operators: host validation/dispatch + HIP kernels
  lib/libcvamd_bench.so -- kernels the benchmark times beside the operators (a copy-bound twin of the
                           fused kernel); nothing in the two libraries above uses it

Usage: python cv-cuda_amd/build.py [--force] [-j N] [--sanitize]
Objects are cached under build/ next to this file and rebuilt when a source or header is newer.

--sanitize builds the same libraries into lib_san/ (objects in build_san/) with AddressSanitizer and
UndefinedBehaviorSanitizer on the HOST code only (device code is compiled as usual). The host logic -
handle pools, reference counts, stride rules, operator validation - can then be run under the sanitizers
without a GPU:

  LD_PRELOAD=$(python cv-cuda_amd/build.py --asan-runtime) ASAN_OPTIONS=detect_leaks=0 \
  CVCUDA_AMD_LIBDIR=cv-cuda_amd/lib_san python -m pytest -m "not gpu" tests/test_core.py tests/test_op_validation.py tests/test_format_api.py tests/test_image_format_api.py -q

(the interpreter itself is not instrumented, so the sanitizer runtime has to be loaded first; leak detection is
off because the interpreter's own allocations would drown the report).
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


def asan_runtime():
    """Path of the AddressSanitizer runtime of hipcc's clang (to LD_PRELOAD into an uninstrumented python)."""
    r = subprocess.run(["hipcc", "-print-file-name=libclang_rt.asan-x86_64.so"], capture_output=True, text=True)
    return r.stdout.strip()


def build(force=False, jobs=8, verbose=True, sanitize=False):
    libdir, objdir = LIBDIR, OBJDIR
    host_extra, hip_extra, link_extra = [], [], []
    if sanitize:
        libdir, objdir = os.path.join(HERE, "lib_san"), os.path.join(HERE, "build_san")
        # on a hipcc line every -fsanitize= goes directly after -Xarch_host: the device pass must not see it
        hip_extra = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined", "-fno-omit-frame-pointer", "-g"]
        host_extra = hip_extra # hipcc compiles the plain .cpp sources as HIP too
        link_extra = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined", "-shared-libsan"]
    os.makedirs(libdir, exist_ok=True)
    os.makedirs(objdir, exist_ok=True)
    newest_header = max(os.path.getmtime(h) for h in _headers())
    core = [(s, host_extra) for s in _sources("nvcv", (".cpp",))]
    ops = [(s, DEVICE + hip_extra if s.endswith(".hip") else host_extra) for s in _sources("cvcuda", (".cpp", ".hip"))]
    bench = [(s, DEVICE + hip_extra) for s in _sources("bench", (".hip",))]
    tasks = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        for group, items in (("nvcv", core), ("cvcuda", ops), ("bench", bench)):
            for src, extra in items:
                obj = os.path.join(objdir, group + "_" + os.path.basename(src) + ".o")
                tasks.append((group, obj, ex.submit(_compile, src, obj, extra, force, newest_header)))
        for group, obj, fut in tasks:
            msgs = fut.result()
            if verbose and msgs:
                print(msgs)
    core_objs = [o for g, o, _ in tasks if g == "nvcv"]
    ops_objs = [o for g, o, _ in tasks if g == "cvcuda"]
    nvcv_so = os.path.join(libdir, "libnvcv_types.so")
    cvcuda_so = os.path.join(libdir, "libcvcuda.so")
    # (the sanitized libraries leave the sanitizer runtime's symbols to the preloaded runtime, so they cannot be
    # linked with --no-undefined)
    link = ["hipcc", "-shared", "-fPIC", "--offload-arch=" + ARCH] + (link_extra if sanitize else ["-Wl,--no-undefined"])
    # ELF symbol versions of the reference's ABI (FUNC@@NVCV_x.y / FUNC@@CVCUDA_x.y), see csrc/abi
    maps = os.path.join(CSRC, "abi")
    subprocess.run(link + core_objs + ["-o", nvcv_so, "-Wl,-soname,libnvcv_types.so",
                                       "-Wl,--version-script=" + os.path.join(maps, "nvcv_types.map")], check=True)
    subprocess.run(link + ops_objs + ["-o", cvcuda_so, "-Wl,-soname,libcvcuda.so", "-L" + libdir, "-lnvcv_types",
                                      "-Wl,-rpath,$ORIGIN",
                                      "-Wl,--version-script=" + os.path.join(maps, "cvcuda.map")], check=True)
    bench_so = os.path.join(libdir, "libcvamd_bench.so")
    subprocess.run(link + [o for g, o, _ in tasks if g == "bench"] + ["-o", bench_so], check=True)
    if not sanitize:
        build_c_caller(libdir)
    return nvcv_so, cvcuda_so, bench_so


def build_c_caller(libdir=LIBDIR):
    """tests/golden/abi_gpu_calls.c -> lib/abi_gpu_calls: a plain C11 program (gcc, the public headers, the HIP
    runtime's C API) that runs three operators through the C ABI; a GPU test runs it and compares what it wrote."""
    src = os.path.join(ROOT, "tests", "golden", "abi_gpu_calls.c")
    exe = os.path.join(libdir, "abi_gpu_calls")
    subprocess.run(["gcc", "-std=c11", "-O1", "-Wall", "-Wextra", "-Werror", "-D__HIP_PLATFORM_AMD__", "-I" + INCLUDE,
                    "-I/opt/rocm/include", src, "-o", exe, "-L" + libdir, "-lcvcuda", "-lnvcv_types", "-L/opt/rocm/lib",
                    "-lamdhip64", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,/opt/rocm/lib"], check=True)
    return exe


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("-j", type=int, default=8)
    ap.add_argument("--sanitize", action="store_true", help="ASan + UBSan build of the host code into lib_san/")
    ap.add_argument("--asan-runtime", action="store_true", help="print the sanitizer runtime to LD_PRELOAD and exit")
    a = ap.parse_args()
    if a.asan_runtime:
        print(asan_runtime())
    else:
        print("\n".join(build(a.force, a.j, sanitize=a.sanitize)))
