/* Operator calls from plain C (C11, gcc) through the C ABI with the HIP runtime's own argument types: the
 * by-value structs (NVCVSize2D, int2, float4), the float[6] matrix, float and bool scalars and the uint32_t
 * flags must arrive as the library's C++ side reads them. Three calls on small images of the recipe
 * value(x, y, c, image) = (x * step + y * 3 + c * 7 + image * 11) & 255 of tests/golden/make_vectors.py:
 *
 *   fused.bin      cvcudaResizeCropConvertReformatSubmit (OpResizeCropConvertReformat.h: NVCVSize2D, int2, two
 *                  floats and a bool after three enumerators)       -> vector fused_linear_f32_nchw
 *   warp.bin       cvcudaWarpAffineSubmit (OpWarpAffine.h: const float[6], int32 flags, border type, float4 by
 *                  value with four different components on RGBA8)   -> vector abi_warp_affine_rgba8_linear
 *   normalize.bin  cvcudaNormalizeSubmit (OpNormalize.h: three floats and uint32_t flags after four handles)
 *                                                                   -> vector normalize_u8_stddev
 *
 * Tensors come from nvcvTensorCalcRequirements + nvcvTensorConstruct (the library's allocator and its row
 * pitch), data moves with hipMemcpy, one packed row at a time. Usage: abi_gpu_calls <output directory>; exits non-zero with a message
 * on any failing call. tests/test_gpu_abi_calls.py compares the files with tests/golden/vectors.npz. */
#include <cvcuda/OpNormalize.h>
#include <cvcuda/OpResizeCropConvertReformat.h>
#include <cvcuda/OpWarpAffine.h>
#include <nvcv/Tensor.h>

#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define CHECK_NVCV(call)                                                                   \
    do                                                                                     \
    {                                                                                      \
        NVCVStatus st_ = (call);                                                           \
        if (st_ != NVCV_SUCCESS)                                                           \
        {                                                                                  \
            char msg_[NVCV_MAX_STATUS_MESSAGE_LENGTH];                                     \
            nvcvGetLastErrorMessage(msg_, (int32_t)sizeof(msg_));                          \
            fprintf(stderr, "%s:%d: %s -> %d (%s)\n", __FILE__, __LINE__, #call, (int)st_, msg_); \
            exit(2);                                                                       \
        }                                                                                  \
    } while (0)

#define CHECK_HIP(call)                                                                                  \
    do                                                                                                   \
    {                                                                                                    \
        hipError_t e_ = (call);                                                                          \
        if (e_ != hipSuccess)                                                                            \
        {                                                                                                \
            fprintf(stderr, "%s:%d: %s -> %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_));      \
            exit(3);                                                                                     \
        }                                                                                                \
    } while (0)

typedef struct
{
    NVCVTensorHandle handle;
    NVCVTensorData   data;
    int              outerDims; /* dimensions before the innermost densely packed run */
    int64_t          rowBytes;  /* bytes of that run */
    int64_t          rows;      /* number of such runs */
} Tensor;

/* A tensor of the given shape from the library's allocator. Its memory is addressed as `rows` densely packed runs
 * (W*C elements of a ...WC layout, W of a planar one) through the exported strides of the dimensions before them. */
static Tensor make_tensor(int rank, const int64_t *shape, NVCVDataType dtype, const char *layout, int elemBytes)
{
    Tensor                 t;
    NVCVTensorLayout       lay;
    NVCVTensorRequirements reqs;
    memset(&t, 0, sizeof(t));
    CHECK_NVCV(nvcvTensorLayoutMake(layout, &lay));
    CHECK_NVCV(nvcvTensorCalcRequirements(rank, shape, dtype, lay, 0, 0, &reqs));
    CHECK_NVCV(nvcvTensorConstruct(&reqs, NULL, &t.handle));
    CHECK_NVCV(nvcvTensorExportData(t.handle, &t.data));
    const int64_t *st = t.data.buffer.strided.strides;
    t.outerDims       = rank - 1;
    while (t.outerDims > 0 && st[t.outerDims - 1] == st[t.outerDims] * shape[t.outerDims])
    {
        --t.outerDims;
    }
    t.rowBytes = elemBytes;
    for (int i = t.outerDims; i < rank; ++i)
    {
        t.rowBytes *= shape[i];
    }
    t.rows = 1;
    for (int i = 0; i < t.outerDims; ++i)
    {
        t.rows *= shape[i];
    }
    return t;
}

/* Byte offset of run r (runs enumerate the outer dimensions in order, the last fastest). */
static int64_t row_offset(const Tensor *t, int64_t r)
{
    int64_t off = 0;
    for (int i = t->outerDims - 1; i >= 0; --i)
    {
        off += (r % t->data.shape[i]) * t->data.buffer.strided.strides[i];
        r /= t->data.shape[i];
    }
    return off;
}

static void upload(const Tensor *t, const void *host)
{
    for (int64_t r = 0; r < t->rows; ++r)
    {
        CHECK_HIP(hipMemcpy((char *)t->data.buffer.strided.basePtr + row_offset(t, r), (const char *)host + r * t->rowBytes,
                            (size_t)t->rowBytes, hipMemcpyHostToDevice));
    }
}

static void download_to_file(const Tensor *t, const char *dir, const char *name)
{
    char path[1024];
    snprintf(path, sizeof(path), "%s/%s", dir, name);
    FILE *f = fopen(path, "wb");
    if (f == NULL)
    {
        fprintf(stderr, "cannot write %s\n", path);
        exit(4);
    }
    char *row = (char *)malloc((size_t)t->rowBytes);
    for (int64_t r = 0; r < t->rows; ++r)
    {
        CHECK_HIP(hipMemcpy(row, (const char *)t->data.buffer.strided.basePtr + row_offset(t, r), (size_t)t->rowBytes,
                            hipMemcpyDeviceToHost));
        fwrite(row, 1, (size_t)t->rowBytes, f);
    }
    free(row);
    fclose(f);
}

static uint8_t *recipe_u8(int n, int h, int w, int c, int step)
{
    uint8_t *p = (uint8_t *)malloc((size_t)n * h * w * c);
    size_t   k = 0;
    for (int i = 0; i < n; ++i)
        for (int y = 0; y < h; ++y)
            for (int x = 0; x < w; ++x)
                for (int ch = 0; ch < c; ++ch)
                    p[k++] = (uint8_t)((x * step + y * 3 + ch * 7 + i * 11) & 255);
    return p;
}

int main(int argc, char **argv)
{
    if (argc != 2)
    {
        fprintf(stderr, "usage: %s <output directory>\n", argv[0]);
        return 1;
    }
    const char *dir = argv[1];
    hipStream_t stream;
    CHECK_HIP(hipSetDevice(0));
    CHECK_HIP(hipStreamCreate(&stream));

    /* ---- fused resize-crop-convert-reformat: 2 x 54 x 96 RGB8 -> resize 46 x 26 -> crop 24 x 24 at (11, 1) -> f32 NCHW */
    {
        const int64_t inShape[4] = {2, 54, 96, 3}, outShape[4] = {2, 3, 24, 24};
        Tensor        in = make_tensor(4, inShape, NVCV_DATA_TYPE_U8, "NHWC", 1);
        Tensor        out = make_tensor(4, outShape, NVCV_DATA_TYPE_F32, "NCHW", 4);
        uint8_t      *src = recipe_u8(2, 54, 96, 3, 5);
        upload(&in, src);
        NVCVOperatorHandle op;
        CHECK_NVCV(cvcudaResizeCropConvertReformatCreate(&op));
        const NVCVSize2D resizeDim = {46, 26};
        const int2       cropPos = {11, 1};
        CHECK_NVCV(cvcudaResizeCropConvertReformatSubmit(op, stream, in.handle, out.handle, resizeDim, NVCV_INTERP_LINEAR,
                                                         cropPos, NVCV_CHANNEL_NO_OP, (float)(1.0 / (255 * 0.226)),
                                                         (float)(-0.449 / 0.226), false));
        CHECK_HIP(hipStreamSynchronize(stream));
        download_to_file(&out, dir, "fused.bin");
        nvcvOperatorDestroy(op);
        nvcvTensorDecRef(in.handle, NULL);
        nvcvTensorDecRef(out.handle, NULL);
        free(src);
    }

    /* ---- affine warp: 1 x 30 x 44 RGBA8, forward map, bilinear, constant border with four different values */
    {
        const int64_t shape[4] = {1, 30, 44, 4};
        Tensor        in = make_tensor(4, shape, NVCV_DATA_TYPE_U8, "NHWC", 1);
        Tensor        out = make_tensor(4, shape, NVCV_DATA_TYPE_U8, "NHWC", 1);
        uint8_t      *src = recipe_u8(1, 30, 44, 4, 5);
        upload(&in, src);
        NVCVOperatorHandle op;
        CHECK_NVCV(cvcudaWarpAffineCreate(&op, 0));
        const NVCVAffineTransform xform = {0.9f, -0.3f, 6.0f, 0.25f, 1.1f, -4.0f};
        const float4              border = {7.f, 80.f, 159.f, 250.f};
        CHECK_NVCV(cvcudaWarpAffineSubmit(op, stream, in.handle, out.handle, xform, NVCV_INTERP_LINEAR, NVCV_BORDER_CONSTANT,
                                          border));
        CHECK_HIP(hipStreamSynchronize(stream));
        download_to_file(&out, dir, "warp.bin");
        nvcvOperatorDestroy(op);
        nvcvTensorDecRef(in.handle, NULL);
        nvcvTensorDecRef(out.handle, NULL);
        free(src);
    }

    /* ---- normalize: 2 x 9 x 14 RGB8, per-channel base and scale, scale is a standard deviation */
    {
        const int64_t shape[4] = {2, 9, 14, 3}, pshape[4] = {1, 1, 1, 3};
        Tensor        in = make_tensor(4, shape, NVCV_DATA_TYPE_U8, "NHWC", 1);
        Tensor        out = make_tensor(4, shape, NVCV_DATA_TYPE_U8, "NHWC", 1);
        Tensor        base = make_tensor(4, pshape, NVCV_DATA_TYPE_F32, "NHWC", 4);
        Tensor        scale = make_tensor(4, pshape, NVCV_DATA_TYPE_F32, "NHWC", 4);
        uint8_t      *src = recipe_u8(2, 9, 14, 3, 7);
        const float   b[3] = {10.0f, 20.0f, 30.0f}, s[3] = {0.5f, 0.25f, 2.0f};
        upload(&in, src);
        upload(&base, b);
        upload(&scale, s);
        NVCVOperatorHandle op;
        CHECK_NVCV(cvcudaNormalizeCreate(&op));
        CHECK_NVCV(cvcudaNormalizeSubmit(op, stream, in.handle, base.handle, scale.handle, out.handle, 40.0f, 100.0f, 0.5f,
                                         CVCUDA_NORMALIZE_SCALE_IS_STDDEV));
        CHECK_HIP(hipStreamSynchronize(stream));
        download_to_file(&out, dir, "normalize.bin");
        nvcvOperatorDestroy(op);
        nvcvTensorDecRef(in.handle, NULL);
        nvcvTensorDecRef(out.handle, NULL);
        nvcvTensorDecRef(base.handle, NULL);
        nvcvTensorDecRef(scale.handle, NULL);
        free(src);
    }
    CHECK_HIP(hipStreamDestroy(stream));
    printf("ok\n");
    return 0;
}
