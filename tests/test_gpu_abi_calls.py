"""Operators called from compiled C on the GPU: cv-cuda_amd/lib/abi_gpu_calls (tests/golden/abi_gpu_calls.c, built by
cv-cuda_amd/build.py with gcc as C11 against the public headers and the HIP runtime's own int2 / float4) runs the fused
operator, WarpAffine and Normalize through the C ABI and writes their raw outputs; they must equal the committed
vectors. This is the by-value argument passing of the reference's interface (cvcuda/OpWarpAffine.h:130-138,
OpResizeCropConvertReformat.h:220-223: NVCVSize2D, int2, float4, float[6], bool) exercised end to end, where the
other GPU tests go through Python's ctypes."""
import os
import subprocess

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "cv-cuda_amd", "lib", "abi_gpu_calls")


def test_operator_calls_from_compiled_c(gpu, tmp_path):
    assert os.path.exists(EXE), "cv-cuda_amd/lib/abi_gpu_calls is missing: run python cv-cuda_amd/build.py"
    r = subprocess.run([EXE, str(tmp_path)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and r.stdout.strip() == "ok", (r.returncode, r.stdout, r.stderr)
    vec = np.load(os.path.join(ROOT, "tests", "golden", "vectors.npz"))
    fused = np.fromfile(tmp_path / "fused.bin", np.float32).reshape(2, 3, 24, 24)
    want = vec["fused_linear_f32_nchw"]
    assert (np.abs(fused - want) <= 1e-5 * np.maximum(1.0, np.abs(want))).all()
    warp = np.fromfile(tmp_path / "warp.bin", np.uint8).reshape(1, 30, 44, 4)
    want = vec["abi_warp_affine_rgba8_linear"]
    np.testing.assert_array_equal(warp, want)
    # every component of the border colour arrived in its channel: the map leaves part of the output uncovered
    border = (warp == np.array([7, 80, 159, 250], np.uint8)).all(axis=-1)
    assert border.any() and not border.all()
    norm = np.fromfile(tmp_path / "normalize.bin", np.uint8).reshape(2, 9, 14, 3)
    np.testing.assert_array_equal(norm, vec["normalize_u8_stddev"])
