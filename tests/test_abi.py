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


# ---- the reference's header-only C++ wrappers, used unchanged -------------------------------------------------
REF = "/root/reference"
REF_NVCV_HPP = os.path.join(REF, "src/nvcv/src/include/nvcv")
REF_CVCUDA_HPP = os.path.join(REF, "src/cvcuda/include/cvcuda")
needs_reference = pytest.mark.skipif(not os.path.isdir(REF_NVCV_HPP), reason="the reference tree is only present in the build container")


def merged_include_tree(dst):
    """include/ of this repository plus the reference's C++ wrapper headers (*.hpp, *.inc), copied at test time into a
    scratch directory: the wrappers include their C headers with quotes, so both must sit in one tree. The operator
    wrappers get the one change a caller makes on this platform: the runtime header and the stream type are HIP's."""
    import shutil
    shutil.copytree(INC, dst)
    for src, sub, patch in ((REF_NVCV_HPP, "nvcv", False), (REF_CVCUDA_HPP, "cvcuda", True)):
        for dp, _, fs in os.walk(src):
            for f in fs:
                if f.endswith((".hpp", ".inc")):
                    out = os.path.join(dst, sub, os.path.relpath(os.path.join(dp, f), src))
                    os.makedirs(os.path.dirname(out), exist_ok=True)
                    text = open(os.path.join(dp, f)).read()
                    if patch:
                        text = text.replace("cuda_runtime.h", "hip/hip_runtime.h").replace("cudaStream_t", "hipStream_t")
                    open(out, "w").write(text)
    return dst


@needs_reference
def test_reference_cpp_wrappers_compile_unchanged(tmp_path):
    """nvcv/*.hpp for every object this library has, and cvcuda/Op*.hpp for every operator it has (reference:
    src/cvcuda/include/cvcuda/OpResizeCropConvertReformat.hpp:63-92 and siblings), in one translation unit."""
    tree = merged_include_tree(str(tmp_path / "inc"))
    ops = sorted(f[:-2] for f in os.listdir(os.path.join(INC, "cvcuda")) if f.startswith("Op") and f.endswith(".h") and f != "Operator.h")
    assert "OpResizeCropConvertReformat" in ops and len(ops) >= 12
    nvcv = ["Tensor", "TensorData", "TensorDataAccess", "TensorLayout", "TensorShape", "Image", "ImageData", "ImageBatch", "ImageBatchData",
            "ImageFormat", "DataType", "DataLayout", "ColorSpec", "Size", "Status", "Exception", "Config", "alloc/Allocator", "alloc/Requirements"]
    tu = tmp_path / "tu.cpp"
    tu.write_text("".join("#include <nvcv/%s.hpp>\n" % h for h in nvcv) + "".join("#include <cvcuda/%s.hpp>\n" % o for o in ops)
                  + "void use(hipStream_t s, cvcuda::ResizeCropConvertReformat &op, const nvcv::Tensor &a, const nvcv::Tensor &b,\n"
                    "         const nvcv::ImageBatchVarShape &batch)\n"
                    "{\n"
                    "    op(s, a, b, NVCVSize2D{455, 256}, NVCV_INTERP_LINEAR, int2{115, 16}, NVCV_CHANNEL_NO_OP, 1.f / 255, 0.f, false);\n"
                    "    op(s, batch, b, NVCVSize2D{455, 256}, NVCV_INTERP_LINEAR, int2{115, 16}, NVCV_CHANNEL_REVERSE, 1.f, 0.f, true);\n"
                    "}\n")
    r = subprocess.run(["hipcc", "-std=c++17", "-fsyntax-only", "--cuda-host-only", "--offload-arch=gfx950", "-Wall", "-I" + tree, str(tu)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-4000:]


HOST_PROGRAM = r"""
#include <nvcv/ColorSpec.hpp>
#include <nvcv/DataType.hpp>
#include <nvcv/Exception.hpp>
#include <nvcv/ImageFormat.hpp>
#include <nvcv/Tensor.hpp>
#include <nvcv/TensorLayout.hpp>
#include <cstdio>
int main()
{
    static_assert(nvcv::FMT_NV12.cvalue() == NVCV_IMAGE_FORMAT_NV12, "constexpr formats");
    constexpr nvcv::ImageFormat made = nvcv::ImageFormat::ConstCreate(nvcv::ColorModel::RGB, nvcv::CSPEC_UNDEFINED, nvcv::MemLayout::PL,
                                                                     nvcv::DataKind::UNSIGNED, nvcv::Swizzle::S_XYZ1, nvcv::Packing::X8_Y8_Z8);
    static_assert(made == nvcv::FMT_RGB8, "constexpr construction");
    nvcv::ImageFormat nv12 = nvcv::FMT_NV12;
    std::printf("planes %d channels %d\n", nv12.numPlanes(), nv12.numChannels());
    std::printf("plane1 %s\n", nvcvDataTypeGetName(nv12.planeDataType(1)));
    nvcv::Size2D half = nv12.planeSize({1920, 1080}, 1);
    std::printf("plane1 size %dx%d\n", half.w, half.h);
    std::printf("edited %s\n", nvcvImageFormatGetName(nv12.memLayout(nvcv::MemLayout::BL).colorSpec(nvcv::CSPEC_BT709).cvalue()));
    std::printf("fourcc %08x\n", nvcv::FMT_YUYV.fourCC());
    std::printf("from planes %d\n", nvcv::ImageFormat::FromPlanes(nv12.planeFormat(0), nv12.planeFormat(1)) == nv12);
    nvcv::DataType t = nvcv::TYPE_3F32;
    std::printf("type %s bpp %d channels %d stride %d\n", nvcvDataTypeGetName(t), t.bitsPerPixel(), t.numChannels(), t.strideBytes());
    std::printf("layout rank %d C at %d\n", nvcv::TENSOR_NHWC.rank(), nvcv::TENSOR_NHWC.find('C'));
    nvcv::Tensor::Requirements req = nvcv::Tensor::CalcRequirements(64, nvcv::Size2D{224, 224}, nvcv::FMT_RGBf32p);
    std::printf("tensor rank %d layout %s strides %lld %lld %lld %lld\n", req.rank, req.layout.data, (long long)req.strides[0],
                (long long)req.strides[1], (long long)req.strides[2], (long long)req.strides[3]);
    try
    {
        nvcv::Tensor::CalcRequirements(nvcv::TensorShape({-4, 2}, "HW"), nvcv::TYPE_U8);
        std::printf("no error\n");
    }
    catch (nvcv::Exception &e)
    {
        std::printf("status %d\n", (int)e.code());
    }
    return 0;
}
"""


@needs_reference
def test_reference_cpp_wrappers_link_and_run_against_the_core_library(cv, tmp_path):
    """A host-only program written against the reference's C++ API (formats, data types, layouts, tensor requirements,
    exceptions) builds with g++ against libnvcv_types.so and prints what the C API's own tests expect."""
    import cvcuda_amd._capi as capi
    libdir = os.path.dirname(capi.nvcv._name)
    tree = merged_include_tree(str(tmp_path / "inc"))
    src = tmp_path / "host.cpp"
    src.write_text(HOST_PROGRAM)
    exe = tmp_path / "host"
    subprocess.run(["g++", "-std=c++17", "-DCVCUDA_NO_HIP_HEADERS", "-I" + tree, str(src), "-L" + libdir, "-lnvcv_types",
                    "-Wl,-rpath," + libdir, "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines()
    assert out == ["planes 2 channels 3",
                   "plane1 NVCV_DATA_TYPE_2U8",
                   "plane1 size 960x540",
                   "edited NVCVImageFormat(YCbCr,BT709,4:2:0,BLOCK2_LINEAR,UNSIGNED,XYZ0,ASSOCIATED,X8,X8_Y8)",
                   "fourcc %08x" % sum(ord(c) << (8 * i) for i, c in enumerate("YUY2")),
                   "from planes 1",
                   "type NVCV_DATA_TYPE_3F32 bpp 96 channels 3 stride 12",
                   "layout rank 4 C at 3",
                   "tensor rank 4 layout NCHW strides 602112 200704 896 4",
                   "status 2"]


VERSION_PROGRAM = r"""
#include <cvcuda/Version.h>
#include <nvcv/Version.h>
#include <stdio.h>
#include <string.h>
#define STR_(a) #a
#define STR(a) STR_(a)
#define CHECK(x) do { if (!(x)) { printf("line %d: %s\n", __LINE__, #x); ++bad; } } while (0)
int main(void)
{
    int bad = 0;
    /* the cases of tests/nvcv_types/system/TestVersion.cpp:25-85 */
    CHECK(NVCV_VERSION == nvcvGetVersion());
    CHECK(NVCV_VERSION_MAJOR == nvcvGetVersion() / 1000000);
    CHECK(NVCV_VERSION_MINOR == nvcvGetVersion() / 10000 % 100);
    CHECK(NVCV_VERSION_PATCH == nvcvGetVersion() / 100 % 100);
    CHECK(NVCV_VERSION_TWEAK == nvcvGetVersion() % 100);
    char want[64];
    snprintf(want, sizeof(want), "%s.%s.%s", STR(NVCV_VERSION_MAJOR), STR(NVCV_VERSION_MINOR), STR(NVCV_VERSION_PATCH));
#if NVCV_VERSION_TWEAK
    strcat(want, "." STR(NVCV_VERSION_TWEAK));
#endif
    if (NVCV_VERSION_SUFFIX[0]) { strcat(want, "-"); strcat(want, NVCV_VERSION_SUFFIX); }
    CHECK(strcmp(want, NVCV_VERSION_STRING) == 0);
    CHECK(1020304 == NVCV_MAKE_VERSION4(1, 2, 3, 4));
    CHECK(1020300 == NVCV_MAKE_VERSION3(1, 2, 3));
    CHECK(1020000 == NVCV_MAKE_VERSION2(1, 2));
    CHECK(1000000 == NVCV_MAKE_VERSION1(1));
    CHECK(NVCV_MAKE_VERSION4(1, 2, 3, 4) == NVCV_MAKE_VERSION(1, 2, 3, 4));
    CHECK(NVCV_MAKE_VERSION4(1, 2, 3, 0) == NVCV_MAKE_VERSION(1, 2, 3));
    CHECK(NVCV_MAKE_VERSION4(1, 2, 0, 0) == NVCV_MAKE_VERSION(1, 2));
    CHECK(NVCV_MAKE_VERSION4(1, 0, 0, 0) == NVCV_MAKE_VERSION(1));
    CHECK(NVCV_VERSION_API == NVCV_MAKE_VERSION(NVCV_VERSION_MAJOR, NVCV_VERSION_MINOR));
    CHECK(NVCV_VERSION_API_IS(NVCV_VERSION_MAJOR, NVCV_VERSION_MINOR));
    CHECK(NVCV_VERSION_API_AT_LEAST(NVCV_VERSION_MAJOR, 0) && !NVCV_VERSION_API_AT_LEAST(NVCV_VERSION_MAJOR + 1, 0));
    CHECK(NVCV_VERSION_API_AT_MOST(NVCV_VERSION_MAJOR + 1, 0) && !NVCV_VERSION_API_AT_MOST(NVCV_VERSION_MAJOR, 0));
    CHECK(NVCV_VERSION_API_IN_RANGE(NVCV_VERSION_MAJOR, 0, NVCV_VERSION_MAJOR, 99));
    /* the operator library carries the same set under its own prefix */
    CHECK(CVCUDA_VERSION == cvcudaGetVersion());
    CHECK(CVCUDA_VERSION == CVCUDA_MAKE_VERSION(CVCUDA_VERSION_MAJOR, CVCUDA_VERSION_MINOR, CVCUDA_VERSION_PATCH));
    CHECK(1020000 == CVCUDA_MAKE_VERSION(1, 2) && 1020304 == CVCUDA_MAKE_VERSION(1, 2, 3, 4));
    CHECK(CVCUDA_VERSION_API_IS(CVCUDA_VERSION_MAJOR, CVCUDA_VERSION_MINOR));
    CHECK(strcmp(CVCUDA_VERSION_STRING, NVCV_VERSION_STRING) == 0);
    return bad;
}
"""


def test_version_macros_and_functions(tmp_path):
    libdir = os.environ.get("CVCUDA_AMD_LIBDIR", os.path.join(ROOT, "cv-cuda_amd", "lib"))
    src = tmp_path / "version.c"
    src.write_text(VERSION_PROGRAM)
    exe = tmp_path / "version"
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", "-DCVCUDA_NO_HIP_HEADERS", "-I" + INC, str(src), "-o", str(exe),
                    "-L" + libdir, "-lcvcuda", "-lnvcv_types", "-Wl,-rpath," + libdir, "-Wl,--allow-shlib-undefined"],
                   check=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
