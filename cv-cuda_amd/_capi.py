"""ctypes declarations of the C ABI in include/nvcv/*.h and include/cvcuda/*.h.

The two shared libraries are loaded from ./lib next to this file; a missing library is an error
(there is no fallback path). torch is imported first so that the HIP runtime already in the
process is the one the libraries bind to.
"""
import ctypes as C
import os

import torch  # noqa: F401  (loads the HIP runtime once, before our libraries resolve it)

_HERE = os.path.dirname(os.path.abspath(__file__))
# CVCUDA_AMD_LIBDIR selects another build of the same libraries (the host-sanitizer build in lib_san/)
_LIBDIR = os.environ.get("CVCUDA_AMD_LIBDIR") or os.path.join(_HERE, "lib")


def _load(name):
    path = os.path.join(_LIBDIR, name)
    if not os.path.exists(path):
        raise ImportError(
            "%s not found: build the native libraries first (python cv-cuda_amd/build.py)" % path)
    return C.CDLL(path, mode=C.RTLD_GLOBAL)


nvcv = _load("libnvcv_types.so")
cvcuda = _load("libcvcuda.so")

NVCV_TENSOR_MAX_RANK = 15
NVCV_MAX_PLANE_COUNT = 6

# status codes ------------------------------------------------------------------------------------
STATUS_NAMES = [
    "NVCV_SUCCESS", "NVCV_ERROR_NOT_IMPLEMENTED", "NVCV_ERROR_INVALID_ARGUMENT",
    "NVCV_ERROR_INVALID_IMAGE_FORMAT", "NVCV_ERROR_INVALID_OPERATION", "NVCV_ERROR_DEVICE",
    "NVCV_ERROR_NOT_READY", "NVCV_ERROR_OUT_OF_MEMORY", "NVCV_ERROR_INTERNAL",
    "NVCV_ERROR_NOT_COMPATIBLE", "NVCV_ERROR_OVERFLOW", "NVCV_ERROR_UNDERFLOW",
]
for _i, _n in enumerate(STATUS_NAMES):
    globals()[_n] = _i


# structs -----------------------------------------------------------------------------------------
class TensorLayout(C.Structure):
    _fields_ = [("data", C.c_char * (NVCV_TENSOR_MAX_RANK + 1)), ("rank", C.c_int32)]

    @classmethod
    def make(cls, s):
        b = s.encode()
        return cls(b, len(b))

    def __str__(self):
        return self.data[:self.rank].decode()


class TensorBufferStrided(C.Structure):
    _fields_ = [("strides", C.c_int64 * NVCV_TENSOR_MAX_RANK), ("basePtr", C.c_void_p)]


class TensorData(C.Structure):
    _fields_ = [("dtype", C.c_uint64), ("layout", TensorLayout), ("rank", C.c_int32),
                ("shape", C.c_int64 * NVCV_TENSOR_MAX_RANK), ("bufferType", C.c_int),
                ("buffer", TensorBufferStrided)]


class MemRequirements(C.Structure):
    _fields_ = [("numBlocks", C.c_int64 * 32)]


class Requirements(C.Structure):
    _fields_ = [("cudaMem", MemRequirements), ("hostMem", MemRequirements), ("hostPinnedMem", MemRequirements)]


class TensorRequirements(C.Structure):
    _fields_ = [("dtype", C.c_uint64), ("layout", TensorLayout), ("rank", C.c_int32),
                ("shape", C.c_int64 * NVCV_TENSOR_MAX_RANK), ("strides", C.c_int64 * NVCV_TENSOR_MAX_RANK),
                ("alignBytes", C.c_int32), ("mem", Requirements)]


class ImagePlaneStrided(C.Structure):
    _fields_ = [("width", C.c_int32), ("height", C.c_int32), ("rowStride", C.c_int32), ("basePtr", C.c_void_p)]


class ImageBufferStrided(C.Structure):
    _fields_ = [("numPlanes", C.c_int32), ("planes", ImagePlaneStrided * NVCV_MAX_PLANE_COUNT)]


class _ImageBufferArr(C.Structure):
    _fields_ = [("numPlanes", C.c_int32), ("planes", C.c_void_p * NVCV_MAX_PLANE_COUNT)]


class ImageBuffer(C.Union):
    _fields_ = [("strided", ImageBufferStrided), ("cudaarray", _ImageBufferArr)]


class ImageData(C.Structure):
    _fields_ = [("format", C.c_uint64), ("bufferType", C.c_int), ("buffer", ImageBuffer)]


class ImageRequirements(C.Structure):
    _fields_ = [("width", C.c_int32), ("height", C.c_int32), ("format", C.c_uint64),
                ("planeRowStride", C.c_int32 * NVCV_MAX_PLANE_COUNT), ("alignBytes", C.c_int32),
                ("mem", Requirements)]


class ImageBatchVarShapeBufferStrided(C.Structure):
    _fields_ = [("uniqueFormat", C.c_uint64), ("maxWidth", C.c_int32), ("maxHeight", C.c_int32),
                ("formatList", C.c_void_p), ("hostFormatList", C.c_void_p), ("imageList", C.c_void_p)]


class ImageBatchData(C.Structure):
    _fields_ = [("numImages", C.c_int32), ("bufferType", C.c_int), ("buffer", ImageBatchVarShapeBufferStrided)]


class ImageBatchVarShapeRequirements(C.Structure):
    _fields_ = [("capacity", C.c_int32), ("alignBytes", C.c_int32), ("mem", Requirements)]


class Size2D(C.Structure):
    _fields_ = [("w", C.c_int32), ("h", C.c_int32)]


class Int2(C.Structure):
    _fields_ = [("x", C.c_int), ("y", C.c_int)]


class RectI(C.Structure):
    _fields_ = [("x", C.c_int32), ("y", C.c_int32), ("width", C.c_int32), ("height", C.c_int32)]


class Float4(C.Structure):
    _fields_ = [("x", C.c_float), ("y", C.c_float), ("z", C.c_float), ("w", C.c_float)]


H = C.c_void_p  # every handle type
ST = C.c_int    # NVCVStatus


def _sig(lib, name, res, *args):
    fn = getattr(lib, name)
    fn.restype = res
    fn.argtypes = list(args)
    return fn


P = C.POINTER
# status
_sig(nvcv, "nvcvStatusGetName", C.c_char_p, ST)
_sig(nvcv, "nvcvGetLastError", ST)
_sig(nvcv, "nvcvGetLastErrorMessage", ST, C.c_char_p, C.c_int32)
_sig(nvcv, "nvcvPeekAtLastError", ST)
_sig(nvcv, "nvcvPeekAtLastErrorMessage", ST, C.c_char_p, C.c_int32)
_sig(nvcv, "nvcvGetVersion", C.c_uint32)
# data type / format queries
for _n in ("nvcvDataTypeGetBitsPerPixel", "nvcvDataTypeGetNumChannels", "nvcvDataTypeGetStrideBytes",
           "nvcvDataTypeGetAlignment"):
    _sig(nvcv, _n, ST, C.c_uint64, P(C.c_int32))
_sig(nvcv, "nvcvDataTypeGetDataKind", ST, C.c_uint64, P(C.c_int))
_sig(nvcv, "nvcvDataTypeGetBitsPerChannel", ST, C.c_uint64, P(C.c_int32 * 4))
_sig(nvcv, "nvcvDataTypeGetName", C.c_char_p, C.c_uint64)
_sig(nvcv, "nvcvDataTypeGetPacking", ST, C.c_uint64, P(C.c_int))
_sig(nvcv, "nvcvMakeDataType", ST, P(C.c_uint64), C.c_int, C.c_int)
_sig(nvcv, "nvcvDataTypeGetChannelType", ST, C.c_uint64, C.c_int32, P(C.c_uint64))
for _n in ("nvcvImageFormatGetNumPlanes", "nvcvImageFormatGetNumChannels"):
    _sig(nvcv, _n, ST, C.c_uint64, P(C.c_int32))
_sig(nvcv, "nvcvImageFormatGetBitsPerChannel", ST, C.c_uint64, P(C.c_int32 * 4))
for _n in ("nvcvImageFormatGetPlaneNumChannels", "nvcvImageFormatGetPlaneBitsPerPixel",
           "nvcvImageFormatGetPlanePixelStrideBytes"):
    _sig(nvcv, _n, ST, C.c_uint64, C.c_int32, P(C.c_int32))
_sig(nvcv, "nvcvImageFormatGetPlanePacking", ST, C.c_uint64, C.c_int32, P(C.c_int))
_sig(nvcv, "nvcvImageFormatGetPlaneDataType", ST, C.c_uint64, C.c_int32, P(C.c_uint64))
_sig(nvcv, "nvcvImageFormatGetPlaneSize", ST, C.c_uint64, C.c_int32, C.c_int32, C.c_int32, P(C.c_int32),
     P(C.c_int32))
for _n in ("nvcvImageFormatGetDataKind", "nvcvImageFormatGetSwizzle", "nvcvImageFormatGetMemLayout",
           "nvcvImageFormatGetColorSpec", "nvcvImageFormatGetColorModel", "nvcvImageFormatGetChromaSubsampling",
           "nvcvImageFormatGetAlphaType"):
    _sig(nvcv, _n, ST, C.c_uint64, P(C.c_int))
_sig(nvcv, "nvcvImageFormatHasSameDataLayout", ST, C.c_uint64, C.c_uint64, P(C.c_int8))
_sig(nvcv, "nvcvImageFormatGetName", C.c_char_p, C.c_uint64)
_sig(nvcv, "nvcvMakeColorImageFormat", ST, P(C.c_uint64), C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
     C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p)
_sig(nvcv, "nvcvMakeYCbCrImageFormat", ST, P(C.c_uint64), C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
     C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p)
_sig(nvcv, "nvcvMakeNonColorImageFormat", ST, P(C.c_uint64), C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
     C.c_int, C.c_int, C.c_void_p)
_sig(nvcv, "nvcvSwizzleGetNumChannels", ST, C.c_int, P(C.c_int32))
_sig(nvcv, "nvcvSwizzleGetChannels", ST, C.c_int, P(C.c_int * 4))
_sig(nvcv, "nvcvMakeSwizzle", ST, P(C.c_int), C.c_int, C.c_int, C.c_int, C.c_int)
_sig(nvcv, "nvcvPackingGetBitsPerPixel", ST, C.c_int, P(C.c_int32))
_sig(nvcv, "nvcvPackingGetNumComponents", ST, C.c_int, P(C.c_int32))
_sig(nvcv, "nvcvPackingGetBitsPerComponent", ST, C.c_int, P(C.c_int32 * 4))
_sig(nvcv, "nvcvChromaSubsamplingGetNumSamples", ST, C.c_int, P(C.c_int32), P(C.c_int32))
# layout
_sig(nvcv, "nvcvTensorLayoutMake", ST, C.c_char_p, P(TensorLayout))
_sig(nvcv, "nvcvTensorLayoutMakeFirst", ST, TensorLayout, C.c_int32, P(TensorLayout))
_sig(nvcv, "nvcvTensorLayoutMakeLast", ST, TensorLayout, C.c_int32, P(TensorLayout))
_sig(nvcv, "nvcvTensorLayoutMakeSubRange", ST, TensorLayout, C.c_int32, C.c_int32, P(TensorLayout))
_sig(nvcv, "nvcvTensorShapePermute", ST, TensorLayout, P(C.c_int64), TensorLayout, P(C.c_int64))
# requirements / allocator
_sig(nvcv, "nvcvRequirementsInit", ST, P(Requirements))
_sig(nvcv, "nvcvRequirementsAdd", ST, P(Requirements), P(Requirements))
_sig(nvcv, "nvcvMemRequirementsCalcTotalSizeBytes", ST, P(MemRequirements), P(C.c_int64))
_sig(nvcv, "nvcvMemRequirementsAddBuffer", ST, P(MemRequirements), C.c_int64, C.c_int64)
MemAllocFunc = C.CFUNCTYPE(C.c_void_p, C.c_void_p, C.c_int64, C.c_int32)
MemFreeFunc = C.CFUNCTYPE(None, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32)


class CustomMemAllocator(C.Structure):
    _fields_ = [("fnAlloc", MemAllocFunc), ("fnFree", MemFreeFunc)]


class ResourceAllocator(C.Structure):
    pass


ResourceAllocatorCleanupFunc = C.CFUNCTYPE(None, C.c_void_p, P(ResourceAllocator))
ResourceAllocator._fields_ = [("ctx", C.c_void_p), ("resType", C.c_int), ("res", CustomMemAllocator),
                              ("cleanup", ResourceAllocatorCleanupFunc)]
_sig(nvcv, "nvcvAllocatorConstructCustom", ST, P(ResourceAllocator), C.c_int32, P(H))
for _t in ("Allocator", "Tensor", "Image", "ImageBatch"):
    for _f in ("DecRef", "IncRef", "RefCount"):
        _sig(nvcv, "nvcv%s%s" % (_t, _f), ST, H, P(C.c_int))
    _sig(nvcv, "nvcv%sSetUserPointer" % _t, ST, H, C.c_void_p)
    _sig(nvcv, "nvcv%sGetUserPointer" % _t, ST, H, P(C.c_void_p))
_sig(nvcv, "nvcvAllocatorAllocHostMemory", ST, H, P(C.c_void_p), C.c_int64, C.c_int32)
_sig(nvcv, "nvcvAllocatorFreeHostMemory", ST, H, C.c_void_p, C.c_int64, C.c_int32)
# tensor
_sig(nvcv, "nvcvTensorCalcRequirements", ST, C.c_int32, P(C.c_int64), C.c_uint64, TensorLayout, C.c_int32,
     C.c_int32, P(TensorRequirements))
_sig(nvcv, "nvcvTensorCalcRequirementsForImages", ST, C.c_int32, C.c_int32, C.c_int32, C.c_uint64, C.c_int32,
     C.c_int32, P(TensorRequirements))
_sig(nvcv, "nvcvTensorConstruct", ST, P(TensorRequirements), H, P(H))
TensorCleanupFunc = C.CFUNCTYPE(None, C.c_void_p, P(TensorData))
_sig(nvcv, "nvcvTensorWrapDataConstruct", ST, P(TensorData), C.c_void_p, C.c_void_p, P(H))
_sig(nvcv, "nvcvTensorWrapImageConstruct", ST, H, P(H))
_sig(nvcv, "nvcvTensorGetDataType", ST, H, P(C.c_uint64))
_sig(nvcv, "nvcvTensorGetLayout", ST, H, P(TensorLayout))
_sig(nvcv, "nvcvTensorGetAllocator", ST, H, P(H))
_sig(nvcv, "nvcvTensorExportData", ST, H, P(TensorData))
_sig(nvcv, "nvcvTensorGetShape", ST, H, P(C.c_int32), P(C.c_int64))
_sig(nvcv, "nvcvTensorReshape", ST, H, C.c_int32, P(C.c_int64), TensorLayout, P(H))
# image
_sig(nvcv, "nvcvImageCalcRequirements", ST, C.c_int32, C.c_int32, C.c_uint64, C.c_int32, C.c_int32,
     P(ImageRequirements))
_sig(nvcv, "nvcvImageConstruct", ST, P(ImageRequirements), H, P(H))
_sig(nvcv, "nvcvImageWrapDataConstruct", ST, P(ImageData), C.c_void_p, C.c_void_p, P(H))
_sig(nvcv, "nvcvImageGetType", ST, H, P(C.c_int))
_sig(nvcv, "nvcvImageGetSize", ST, H, P(C.c_int32), P(C.c_int32))
_sig(nvcv, "nvcvImageGetFormat", ST, H, P(C.c_uint64))
_sig(nvcv, "nvcvImageGetAllocator", ST, H, P(H))
_sig(nvcv, "nvcvImageExportData", ST, H, P(ImageData))
# image batch
_sig(nvcv, "nvcvImageBatchVarShapeCalcRequirements", ST, C.c_int32, P(ImageBatchVarShapeRequirements))
_sig(nvcv, "nvcvImageBatchVarShapeConstruct", ST, P(ImageBatchVarShapeRequirements), H, P(H))
_sig(nvcv, "nvcvImageBatchGetType", ST, H, P(C.c_int))
_sig(nvcv, "nvcvImageBatchGetCapacity", ST, H, P(C.c_int32))
_sig(nvcv, "nvcvImageBatchGetNumImages", ST, H, P(C.c_int32))
_sig(nvcv, "nvcvImageBatchGetAllocator", ST, H, P(H))
_sig(nvcv, "nvcvImageBatchExportData", ST, H, C.c_void_p, P(ImageBatchData))
_sig(nvcv, "nvcvImageBatchVarShapeGetMaxSize", ST, H, P(C.c_int32), P(C.c_int32))
_sig(nvcv, "nvcvImageBatchVarShapeGetUniqueFormat", ST, H, P(C.c_uint64))
_sig(nvcv, "nvcvImageBatchVarShapePushImages", ST, H, P(H), C.c_int32)
PushImageFunc = C.CFUNCTYPE(C.c_void_p, C.c_void_p)
_sig(nvcv, "nvcvImageBatchVarShapePushImagesCallback", ST, H, PushImageFunc, C.c_void_p)
_sig(nvcv, "nvcvImageBatchVarShapePopImages", ST, H, C.c_int32)
_sig(nvcv, "nvcvImageBatchVarShapeClear", ST, H)
_sig(nvcv, "nvcvImageBatchVarShapeGetImages", ST, H, C.c_int32, P(H), C.c_int32)
for _n in ("nvcvConfigSetMaxImageCount", "nvcvConfigSetMaxImageBatchCount", "nvcvConfigSetMaxTensorCount",
           "nvcvConfigSetMaxAllocatorCount"):
    _sig(nvcv, _n, ST, C.c_int32)

# operators (stream slot: hipStream_t as void*)
_sig(cvcuda, "nvcvOperatorDestroy", None, H)
_sig(cvcuda, "cvcudaGetVersion", C.c_uint32)
_sig(cvcuda, "cvcudaResizeCropConvertReformatCreate", ST, P(H))
_sig(cvcuda, "cvcudaResizeCropConvertReformatSubmit", ST, H, C.c_void_p, H, H, Size2D, C.c_int, Int2, C.c_int,
     C.c_float, C.c_float, C.c_bool)
_sig(cvcuda, "cvcudaResizeCropConvertReformatVarShapeSubmit", ST, H, C.c_void_p, H, H, Size2D, C.c_int, Int2,
     C.c_int, C.c_float, C.c_float, C.c_bool)


class ChannelNormalize(C.Structure):
    """CVCUDAXChannelNormalize (cvcuda/OpResizeCropConvertReformat.h, extension)."""
    _fields_ = [("base", C.c_float * 3), ("scale", C.c_float * 3), ("globalScale", C.c_float), ("shift", C.c_float),
                ("epsilon", C.c_float), ("flags", C.c_uint32)]


_sig(cvcuda, "cvcudaxResizeCropConvertReformatNormalizeSubmit", ST, H, C.c_void_p, H, H, Size2D, C.c_int, Int2,
     C.c_int, C.c_float, C.c_float, C.c_bool, P(ChannelNormalize))
_sig(cvcuda, "cvcudaxResizeCropConvertReformatNormalizeVarShapeSubmit", ST, H, C.c_void_p, H, H, Size2D, C.c_int,
     Int2, C.c_int, C.c_float, C.c_float, C.c_bool, P(ChannelNormalize))

_sig(cvcuda, "cvcudaCropFlipNormalizeReformatCreate", ST, P(H))
_sig(cvcuda, "cvcudaCropFlipNormalizeReformatSubmit", ST, H, C.c_void_p, H, H, H, C.c_int, C.c_float, H, H, H,
     C.c_float, C.c_float, C.c_float, C.c_uint32)
_sig(cvcuda, "cvcudaConvertToCreate", ST, P(H))
_sig(cvcuda, "cvcudaConvertToSubmit", ST, H, C.c_void_p, H, H, C.c_double, C.c_double)
_sig(cvcuda, "cvcudaCustomCropCreate", ST, P(H))
_sig(cvcuda, "cvcudaCustomCropSubmit", ST, H, C.c_void_p, H, H, RectI)
_sig(cvcuda, "cvcudaCenterCropCreate", ST, P(H))
_sig(cvcuda, "cvcudaCenterCropSubmit", ST, H, C.c_void_p, H, H, C.c_int32, C.c_int32)
_sig(cvcuda, "cvcudaFlipCreate", ST, P(H), C.c_int32)
_sig(cvcuda, "cvcudaFlipSubmit", ST, H, C.c_void_p, H, H, C.c_int32)
_sig(cvcuda, "cvcudaFlipVarShapeSubmit", ST, H, C.c_void_p, H, H, H)


def declare_optional(name, res, *args):
    """Declares an operator entry point if the library exports it; returns whether it does."""
    if hasattr(cvcuda, name):
        _sig(cvcuda, name, res, *args)
        return True
    return False


declare_optional("cvcudaResizeCreate", ST, P(H))
declare_optional("cvcudaResizeSubmit", ST, H, C.c_void_p, H, H, C.c_int)
declare_optional("cvcudaResizeVarShapeSubmit", ST, H, C.c_void_p, H, H, C.c_int)
declare_optional("cvcudaCvtColorCreate", ST, P(H))
declare_optional("cvcudaCvtColorSubmit", ST, H, C.c_void_p, H, H, C.c_int)
declare_optional("cvcudaCvtColorVarShapeSubmit", ST, H, C.c_void_p, H, H, C.c_int)
declare_optional("cvcudaNormalizeCreate", ST, P(H))
declare_optional("cvcudaNormalizeSubmit", ST, H, C.c_void_p, H, H, H, H, C.c_float, C.c_float, C.c_float,
                 C.c_uint32)
declare_optional("cvcudaNormalizeVarShapeSubmit", ST, H, C.c_void_p, H, H, H, H, C.c_float, C.c_float,
                 C.c_float, C.c_uint32)
declare_optional("cvcudaReformatCreate", ST, P(H))
declare_optional("cvcudaReformatSubmit", ST, H, C.c_void_p, H, H)
declare_optional("cvcudaWarpAffineCreate", ST, P(H), C.c_int32)
declare_optional("cvcudaWarpAffineSubmit", ST, H, C.c_void_p, H, H, P(C.c_float), C.c_int32, C.c_int, Float4)
declare_optional("cvcudaWarpAffineVarShapeSubmit", ST, H, C.c_void_p, H, H, H, C.c_int32, C.c_int, Float4)
declare_optional("cvcudaWarpPerspectiveCreate", ST, P(H), C.c_int32)
declare_optional("cvcudaWarpPerspectiveSubmit", ST, H, C.c_void_p, H, H, P(C.c_float), C.c_int32, C.c_int, Float4)
declare_optional("cvcudaWarpPerspectiveVarShapeSubmit", ST, H, C.c_void_p, H, H, H, C.c_int32, C.c_int, Float4)
