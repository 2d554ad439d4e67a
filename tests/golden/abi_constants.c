/* Prints the numeric value of ABI-relevant constants and the size / field offsets of the plain-data
 * structs of the NVCV C headers found on the include path. Compiled once against the reference's
 * headers (make_abi_constants.sh, output committed as abi_constants.txt) and, by the test-suite,
 * against this repository's headers; both outputs must be identical. */
#include <stddef.h>
#include <stdio.h>

#include <nvcv/BorderType.h>
#include <nvcv/ImageBatch.h>
#include <nvcv/Size.h>
#include <nvcv/Tensor.h>

#define V(x) printf(#x " %llu\n", (unsigned long long)(x))
#define S(t) printf("sizeof(" #t ") %zu\n", sizeof(t))
#define O(t, f) printf("offsetof(" #t "," #f ") %zu\n", offsetof(t, f))

int main(void)
{
#include "abi_constants_all.inc"
#include "abi_detail_macros.inc"
    V(NVCV_IMAGE_FORMAT_U8);
    V(NVCV_IMAGE_FORMAT_S8);
    V(NVCV_IMAGE_FORMAT_U16);
    V(NVCV_IMAGE_FORMAT_S16);
    V(NVCV_IMAGE_FORMAT_U32);
    V(NVCV_IMAGE_FORMAT_S32);
    V(NVCV_IMAGE_FORMAT_F16);
    V(NVCV_IMAGE_FORMAT_F32);
    V(NVCV_IMAGE_FORMAT_F64);
    V(NVCV_IMAGE_FORMAT_2S16);
    V(NVCV_IMAGE_FORMAT_2F32);
    V(NVCV_IMAGE_FORMAT_Y8);
    V(NVCV_IMAGE_FORMAT_Y8_ER);
    V(NVCV_IMAGE_FORMAT_NV12);
    V(NVCV_IMAGE_FORMAT_NV12_ER);
    V(NVCV_IMAGE_FORMAT_NV21);
    V(NVCV_IMAGE_FORMAT_NV21_ER);
    V(NVCV_IMAGE_FORMAT_UYVY);
    V(NVCV_IMAGE_FORMAT_YUYV);
    V(NVCV_IMAGE_FORMAT_YUV8p);
    V(NVCV_IMAGE_FORMAT_RGB8);
    V(NVCV_IMAGE_FORMAT_BGR8);
    V(NVCV_IMAGE_FORMAT_RGBA8);
    V(NVCV_IMAGE_FORMAT_BGRA8);
    V(NVCV_IMAGE_FORMAT_RGBf32);
    V(NVCV_IMAGE_FORMAT_BGRf32);
    V(NVCV_IMAGE_FORMAT_RGBAf32);
    V(NVCV_IMAGE_FORMAT_BGRAf32);
    V(NVCV_IMAGE_FORMAT_RGBf16);
    V(NVCV_IMAGE_FORMAT_BGRf16);
    V(NVCV_IMAGE_FORMAT_RGBAf16);
    V(NVCV_IMAGE_FORMAT_BGRAf16);
    V(NVCV_IMAGE_FORMAT_HSV8);
    V(NVCV_IMAGE_FORMAT_RGB8p);
    V(NVCV_IMAGE_FORMAT_BGR8p);
    V(NVCV_IMAGE_FORMAT_RGBA8p);
    V(NVCV_IMAGE_FORMAT_BGRA8p);
    V(NVCV_IMAGE_FORMAT_RGBf32p);
    V(NVCV_IMAGE_FORMAT_BGRf32p);
    V(NVCV_IMAGE_FORMAT_RGBAf32p);
    V(NVCV_IMAGE_FORMAT_BGRAf32p);
    V(NVCV_IMAGE_FORMAT_RGBf16p);
    V(NVCV_IMAGE_FORMAT_BGRf16p);
    V(NVCV_DATA_TYPE_U8);
    V(NVCV_DATA_TYPE_2U8);
    V(NVCV_DATA_TYPE_3U8);
    V(NVCV_DATA_TYPE_4U8);
    V(NVCV_DATA_TYPE_S8);
    V(NVCV_DATA_TYPE_U16);
    V(NVCV_DATA_TYPE_3U16);
    V(NVCV_DATA_TYPE_S16);
    V(NVCV_DATA_TYPE_4S16);
    V(NVCV_DATA_TYPE_U32);
    V(NVCV_DATA_TYPE_S32);
    V(NVCV_DATA_TYPE_F16);
    V(NVCV_DATA_TYPE_F32);
    V(NVCV_DATA_TYPE_2F32);
    V(NVCV_DATA_TYPE_3F32);
    V(NVCV_DATA_TYPE_4F32);
    V(NVCV_DATA_TYPE_F64);
    V(NVCV_DATA_TYPE_4F64);
    V(NVCV_DATA_TYPE_U64);
    V(NVCV_DATA_TYPE_S64);
    V(NVCV_DATA_TYPE_C64);
    V(NVCV_DATA_TYPE_2C128);
    V(NVCV_PACKING_X8);
    V(NVCV_PACKING_X8_Y8_Z8);
    V(NVCV_PACKING_X8_Y8_Z8_W8);
    V(NVCV_PACKING_X32_Y32_Z32);
    V(NVCV_PACKING_X8_Y8__X8_Z8);
    V(NVCV_PACKING_Y8_X8__Z8_X8);
    V(NVCV_PACKING_X64_Y64_Z64_W64);
    V(NVCV_PACKING_X10Y10Z10W2);
    V(NVCV_PACKING_X32_Y24b8);
    V(NVCV_COLOR_SPEC_BT601);
    V(NVCV_COLOR_SPEC_BT601_ER);
    V(NVCV_COLOR_SPEC_sRGB);
    V(NVCV_COLOR_SPEC_DISPLAYP3_LINEAR);
    V(NVCV_SUCCESS);
    V(NVCV_ERROR_NOT_IMPLEMENTED);
    V(NVCV_ERROR_INVALID_ARGUMENT);
    V(NVCV_ERROR_INVALID_IMAGE_FORMAT);
    V(NVCV_ERROR_INVALID_OPERATION);
    V(NVCV_ERROR_DEVICE);
    V(NVCV_ERROR_NOT_READY);
    V(NVCV_ERROR_OUT_OF_MEMORY);
    V(NVCV_ERROR_INTERNAL);
    V(NVCV_ERROR_NOT_COMPATIBLE);
    V(NVCV_ERROR_OVERFLOW);
    V(NVCV_ERROR_UNDERFLOW);
    V(NVCV_BORDER_CONSTANT);
    V(NVCV_BORDER_REPLICATE);
    V(NVCV_BORDER_REFLECT);
    V(NVCV_BORDER_WRAP);
    V(NVCV_BORDER_REFLECT101);
    V(NVCV_SWIZZLE_XYZW);
    V(NVCV_SWIZZLE_ZYX1);
    V(NVCV_SWIZZLE_0ZXY);
    V(NVCV_SWIZZLE_XYZ1);
    V(NVCV_SWIZZLE_YZW0);
    V(NVCV_CSS_420);
    V(NVCV_CSS_422);
    V(NVCV_CSS_410R);
    V(NVCV_COLOR_MODEL_HSV);
    V(NVCV_COLOR_MODEL_YCCK);
    V(NVCV_TENSOR_BUFFER_STRIDED_CUDA);
    V(NVCV_IMAGE_BUFFER_STRIDED_CUDA);
    V(NVCV_IMAGE_BATCH_VARSHAPE_BUFFER_STRIDED_CUDA);
    V(NVCV_RESOURCE_MEM_HOST);
    V(NVCV_RESOURCE_MEM_CUDA);
    V(NVCV_RESOURCE_MEM_HOST_PINNED);
    V(NVCV_TYPE_IMAGE_WRAPDATA);
    V(NVCV_TYPE_IMAGEBATCH_VARSHAPE);
    V(NVCV_MAX_PLANE_COUNT);
    V(NVCV_TENSOR_MAX_RANK);
    V(NVCV_MAX_MEM_REQUIREMENTS_LOG2_BLOCK_SIZE);
    V(NVCV_MAX_STATUS_MESSAGE_LENGTH);
    S(NVCVTensorLayout);
    S(NVCVTensorBufferStrided);
    S(NVCVTensorData);
    S(NVCVTensorRequirements);
    S(NVCVImagePlaneStrided);
    S(NVCVImageBufferStrided);
    S(NVCVImageData);
    S(NVCVImageRequirements);
    S(NVCVImageBatchVarShapeBufferStrided);
    S(NVCVImageBatchData);
    S(NVCVImageBatchVarShapeRequirements);
    S(NVCVMemRequirements);
    S(NVCVRequirements);
    S(NVCVResourceAllocator);
    S(NVCVSize2D);
    S(NVCVPackingParams);
    O(NVCVTensorLayout, rank);
    O(NVCVTensorData, layout);
    O(NVCVTensorData, rank);
    O(NVCVTensorData, shape);
    O(NVCVTensorData, bufferType);
    O(NVCVTensorData, buffer);
    O(NVCVTensorBufferStrided, basePtr);
    O(NVCVTensorRequirements, strides);
    O(NVCVTensorRequirements, alignBytes);
    O(NVCVTensorRequirements, mem);
    O(NVCVImagePlaneStrided, basePtr);
    O(NVCVImageBufferStrided, planes);
    O(NVCVImageData, bufferType);
    O(NVCVImageData, buffer);
    O(NVCVImageRequirements, format);
    O(NVCVImageRequirements, planeRowStride);
    O(NVCVImageRequirements, alignBytes);
    O(NVCVImageRequirements, mem);
    O(NVCVImageBatchVarShapeBufferStrided, maxWidth);
    O(NVCVImageBatchVarShapeBufferStrided, formatList);
    O(NVCVImageBatchVarShapeBufferStrided, imageList);
    O(NVCVImageBatchData, bufferType);
    O(NVCVImageBatchData, buffer);
    O(NVCVImageBatchVarShapeRequirements, mem);
    O(NVCVRequirements, hostMem);
    O(NVCVRequirements, hostPinnedMem);
    O(NVCVResourceAllocator, resType);
    O(NVCVResourceAllocator, res);
    O(NVCVResourceAllocator, cleanup);
    return 0;
}
