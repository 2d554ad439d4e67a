"""The host logic of the two libraries (handle pools, reference counts, stride rules, operator validation) under
AddressSanitizer and UndefinedBehaviorSanitizer: builds cv-cuda_amd/lib_san (host code instrumented, device code
as usual) and runs the host-side test files against it in a child interpreter with the sanitizer runtime
preloaded. No GPU is involved: those tests stop at validation or use fake device addresses.
The handle pools are also run under ThreadSanitizer, from a C program whose threads create, share and destroy
objects (tests/golden/handle_pool_stress.c)."""
import glob
import importlib.util
import os
import shutil
import subprocess
import sys
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "cv-cuda_amd")


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc to build the instrumented libraries")
def test_core_and_validation_are_clean_under_asan_and_ubsan():
    spec = importlib.util.spec_from_file_location("_cvbuild_san", os.path.join(PKG, "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod.build(sanitize=True, verbose=False)
    runtime = mod.asan_runtime()
    assert os.path.exists(runtime), runtime
    with tempfile.TemporaryDirectory() as logs:
        env = dict(os.environ)
        env["LD_PRELOAD"] = runtime + (":" + env["LD_PRELOAD"] if env.get("LD_PRELOAD") else "")
        env["ASAN_OPTIONS"] = "detect_leaks=0:log_path=" + os.path.join(logs, "asan")
        env["UBSAN_OPTIONS"] = "print_stacktrace=1:log_path=" + os.path.join(logs, "ubsan")
        env["CVCUDA_AMD_LIBDIR"] = os.path.join(PKG, "lib_san")
        r = subprocess.run([sys.executable, "-m", "pytest", "-q", "-x", "-m", "not gpu", "-p", "no:cacheprovider",
                            os.path.join(ROOT, "tests", "test_core.py"), os.path.join(ROOT, "tests", "test_op_validation.py"),
                            os.path.join(ROOT, "tests", "test_format_api.py"), os.path.join(ROOT, "tests", "test_image_format_api.py")],
                           env=env, capture_output=True, text=True, timeout=900)
        reports = []
        for f in glob.glob(os.path.join(logs, "*")):
            reports.append(open(f).read()[:4000])
        assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:] + "".join(reports)
        assert not reports, "sanitizer reports:\n" + "\n".join(reports)


@pytest.mark.skipif(shutil.which("hipcc") is None or shutil.which("amdclang") is None,
                    reason="needs hipcc and amdclang to build the instrumented core library")
def test_handle_pools_are_clean_under_thread_sanitizer(tmp_path):
    """Builds the core library (host code only) and the threaded C program with -fsanitize=thread; the program is
    linked by the C++ driver so that the run time also sees the guards of function-local statics."""
    csrc = os.path.join(PKG, "csrc")
    inc = os.path.join(ROOT, "include")
    objs, procs = [], []
    for src in sorted(glob.glob(os.path.join(csrc, "nvcv", "*.cpp"))):
        obj = str(tmp_path / (os.path.basename(src) + ".o"))
        objs.append(obj)
        procs.append(subprocess.Popen(["hipcc", "-std=c++17", "-O1", "-g", "-fPIC", "-fvisibility=hidden", "-I" + inc,
                                       "-I" + csrc, "-Xarch_host", "-fsanitize=thread", "-c", src, "-o", obj],
                                      stdout=subprocess.DEVNULL, stderr=subprocess.PIPE, text=True))
    for p in procs:
        err = p.communicate()[1]
        assert p.returncode == 0, err[-3000:]
    lib = str(tmp_path / "libnvcv_types.so")
    subprocess.run(["hipcc", "-shared", "-fPIC", "-Xarch_host", "-fsanitize=thread"] + objs
                   + ["-o", lib, "-Wl,-soname,libnvcv_types.so",
                      "-Wl,--version-script=" + os.path.join(csrc, "abi", "nvcv_types.map")], check=True)
    obj = str(tmp_path / "stress.o")
    subprocess.run(["amdclang", "-std=c11", "-g", "-fsanitize=thread", "-D_POSIX_C_SOURCE=200112L",
                    "-DCVCUDA_NO_HIP_HEADERS", "-I" + inc, "-c",
                    os.path.join(ROOT, "tests", "golden", "handle_pool_stress.c"), "-o", obj], check=True)
    exe = str(tmp_path / "stress")
    subprocess.run(["amdclang++", "-fsanitize=thread", obj, "-o", exe, "-pthread", "-L" + str(tmp_path), "-lnvcv_types",
                    "-Wl,-rpath," + str(tmp_path)], check=True)
    r = subprocess.run([exe, "8", "2000"], capture_output=True, text=True, timeout=600)
    out = r.stdout + r.stderr
    assert r.returncode == 0 and "ThreadSanitizer" not in out and r.stdout.strip().endswith(" 0 failed"), out[-6000:]
