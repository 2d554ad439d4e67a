"""The host logic of the two libraries (handle pools, reference counts, stride rules, operator validation) under
AddressSanitizer and UndefinedBehaviorSanitizer: builds cv-cuda_amd/lib_san (host code instrumented, device code
as usual) and runs the host-side test files against it in a child interpreter with the sanitizer runtime
preloaded. No GPU is involved: those tests stop at validation or use fake device addresses."""
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
