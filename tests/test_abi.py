"""C-ABI checks that need no GPU: constants and struct layouts equal the reference's (golden fixture
generated from the reference's own headers by tests/golden/make_abi_constants.sh), the libraries load,
and every function declared in include/ is exported."""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include")
GOLD = os.path.join(ROOT, "tests", "golden")


def test_constants_and_layouts_match_reference_headers(tmp_path):
    exe = tmp_path / "abi"
    subprocess.run(["gcc", "-std=c11", "-DCVCUDA_NO_HIP_HEADERS", "-I" + INC, os.path.join(GOLD, "abi_constants.c"),
                    "-o", str(exe)], check=True)
    got = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    want = open(os.path.join(GOLD, "abi_constants.txt")).read()
    assert got == want


def test_headers_compile_as_c_and_cpp(tmp_path):
    hdrs = []
    for sub in ("nvcv", "nvcv/alloc", "cvcuda"):
        d = os.path.join(INC, sub)
        hdrs += ["%s/%s" % (sub, f) for f in sorted(os.listdir(d)) if f.endswith(".h")]
    src = tmp_path / "all.c"
    src.write_text("".join("#include <%s>\n" % h for h in hdrs) + "int main(void){return 0;}\n")
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", "-DCVCUDA_NO_HIP_HEADERS", "-I" + INC, "-c", str(src),
                    "-o", str(tmp_path / "c.o")], check=True)
    subprocess.run(["g++", "-std=c++17", "-x", "c++", "-Wall", "-Werror", "-DCVCUDA_NO_HIP_HEADERS", "-I" + INC, "-c",
                    str(src), "-o", str(tmp_path / "cpp.o")], check=True)


def declared_functions():
    names = {}
    for dp, _, fs in os.walk(INC):
        for f in fs:
            if not f.endswith(".h"):
                continue
            text = open(os.path.join(dp, f)).read()
            text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
            text = "\n".join(l for l in text.splitlines() if not l.lstrip().startswith("#"))
            for m in re.finditer(r"\b(NVCV_PUBLIC|CVCUDA_PUBLIC)\b[^;{]*?\b(\w+)\s*\(", text):
                names[m.group(2)] = "nvcv" if m.group(1) == "NVCV_PUBLIC" else "cvcuda"
    return names


def test_every_declared_function_is_exported(cv):
    import cvcuda_amd._capi as capi
    libs = {"nvcv": capi.nvcv, "cvcuda": capi.cvcuda}
    decl = declared_functions()
    assert len(decl) > 100
    missing = [n for n, lib in sorted(decl.items()) if not hasattr(libs[lib], n)]
    assert not missing, "declared in include/ but not exported: %s" % missing


def test_versions(cv):
    import cvcuda_amd._capi as capi
    assert capi.nvcv.nvcvGetVersion() == 150000
    assert capi.cvcuda.cvcudaGetVersion() == 150000


def test_by_value_struct_arguments_from_plain_c(cv, tmp_path):
    """A C caller (no HIP headers, stand-in int2/NVCVSize2D) passes the by-value structs; the values
    must arrive intact -- observed through the error messages that echo them."""
    libdir = os.path.join(ROOT, "cv-cuda_amd", "lib")
    src = tmp_path / "byval.c"
    src.write_text(r'''
#define CVCUDA_NO_HIP_HEADERS
#include <cvcuda/OpResizeCropConvertReformat.h>
#include <stdio.h>
#include <string.h>
static NVCVTensorHandle wrap(int n, int h, int w, int c, NVCVDataType dt, const char *layout, int es) {
    NVCVTensorData d; memset(&d, 0, sizeof(d));
    d.dtype = dt; nvcvTensorLayoutMake(layout, &d.layout); d.rank = 4;
    int64_t shape[4] = {n, h, w, c};
    if (layout[1] == 'C') { shape[1] = c; shape[2] = h; shape[3] = w; }
    int64_t st = es;
    for (int i = 3; i >= 0; --i) { d.shape[i] = shape[i]; d.buffer.strided.strides[i] = st; st *= shape[i]; }
    d.bufferType = NVCV_TENSOR_BUFFER_STRIDED_CUDA; d.buffer.strided.basePtr = (NVCVByte *)0x10000;
    NVCVTensorHandle h_ = NULL;
    if (nvcvTensorWrapDataConstruct(&d, NULL, NULL, &h_) != NVCV_SUCCESS) return NULL;
    return h_;
}
int main(void) {
    NVCVOperatorHandle op; char msg[256];
    if (cvcudaResizeCropConvertReformatCreate(&op) != NVCV_SUCCESS) return 1;
    NVCVTensorHandle in = wrap(2, 40, 50, 3, NVCV_DATA_TYPE_U8, "NHWC", 1);
    NVCVTensorHandle out = wrap(2, 10, 12, 3, NVCV_DATA_TYPE_F32, "NCHW", 4);
    if (!in || !out) return 2;
    NVCVSize2D rs = {33, 1}; int2 crop = {7, 9};
    NVCVStatus st = cvcudaResizeCropConvertReformatSubmit(op, NULL, in, out, rs, NVCV_INTERP_LINEAR, crop,
                                                          NVCV_CHANNEL_NO_OP, 1.f, 0.f, false);
    nvcvGetLastErrorMessage(msg, sizeof(msg)); printf("%d|%s\n", (int)st, msg);
    rs.w = 20; rs.h = 30; crop.x = 11; crop.y = 22;
    st = cvcudaResizeCropConvertReformatSubmit(op, NULL, in, out, rs, NVCV_INTERP_LINEAR, crop, NVCV_CHANNEL_NO_OP,
                                               1.f, 0.f, false);
    nvcvGetLastErrorMessage(msg, sizeof(msg)); printf("%d|%s\n", (int)st, msg);
    rs.w = 40; rs.h = 40; crop.x = 1; crop.y = 2;
    st = cvcudaResizeCropConvertReformatSubmit(op, NULL, in, out, rs, NVCV_INTERP_CUBIC, crop, NVCV_CHANNEL_NO_OP,
                                               1.f, 0.f, false);
    nvcvGetLastErrorMessage(msg, sizeof(msg)); printf("%d|%s\n", (int)st, msg);
    nvcvTensorDecRef(in, NULL); nvcvTensorDecRef(out, NULL); nvcvOperatorDestroy(op);
    return 0;
}
''')
    exe = tmp_path / "byval"
    subprocess.run(["gcc", "-std=c11", "-I" + INC, str(src), "-o", str(exe), "-L" + libdir, "-lcvcuda", "-lnvcv_types",
                    "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib"], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines()
    assert out[0].startswith("2|Invalid resize dimensions: width x hight = 33 x 1")
    assert out[1].startswith("2|Invalid crop region: crop region(x, y, w, h) = (11, 22, 12, 10)")
    assert out[2] == "2|Interpolation not implemented: NVCV_INTERP_CUBIC"


def test_symbol_versions_match_reference_tags(cv):
    """Exported functions carry the ELF symbol versions the reference gives them (NVCV_PROJ_DEFINE_API,
    src/nvcv/util/SymbolVersioning.hpp:69-92), so binaries linked against the reference resolve."""
    import os
    import re
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for lib, mapfile in (("libcvcuda.so", "cvcuda.map"), ("libnvcv_types.so", "nvcv_types.map")):
        text = open(os.path.join(root, "cv-cuda_amd", "csrc", "abi", mapfile)).read()
        want = {}
        for node, body in re.findall(r"(\w+_\d+\.\d+)\s*\{\s*global:(.*?)\};", text, re.S):
            for f in re.findall(r"(\w+);", body):
                want[f] = node
        out = subprocess.run(["nm", "-D", "--with-symbol-versions", os.path.join(root, "cv-cuda_amd", "lib", lib)],
                             capture_output=True, text=True, check=True).stdout
        have = dict(re.findall(r" T (\w+)@@(\w+\.\d+)", out))
        assert len(want) > 20
        for f, node in want.items():
            assert have.get(f) == node, (f, node, have.get(f))
    # spot values read from the reference's sources
    assert "cvcudaResizeCropConvertReformatSubmit@@CVCUDA_0.10" in subprocess.run(
        ["nm", "-D", "--with-symbol-versions", os.path.join(root, "cv-cuda_amd", "lib", "libcvcuda.so")],
        capture_output=True, text=True).stdout
