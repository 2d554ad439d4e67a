/* Argument-checking behaviour of the core objects, written in plain C against the public headers. The rows are the
 * cases of the reference's own unit tests (which status each bad call returns):
 *   tests/nvcv_types/system/TestTensor.cpp:58-447 (shapes and strides) and 529-760, TestImage.cpp:267-515, TestImageBatch.cpp:359-694,
 *   TestAllocatorC.cpp:33-135 and 224-402, TestConfig.cpp:107-131.
 * Tensors and images are built on a custom allocator that serves "device" memory from the host heap, so the first
 * part runs without a GPU. `device` as first argument adds the image-batch cases, whose construction needs one.
 * Prints one line per failed check and exits with their count. */
#include <nvcv/Config.h>
#include <nvcv/Image.h>
#include <nvcv/ImageBatch.h>
#include <nvcv/Tensor.h>
#include <nvcv/TensorShape.h>
#include <nvcv/alloc/Allocator.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static int g_failed = 0;

#define EXPECT(want, call)                                                                        \
    do                                                                                            \
    {                                                                                             \
        long long got_ = (long long)(call);                                                       \
        if (got_ != (long long)(want))                                                            \
        {                                                                                         \
            printf("line %d: %s -> %lld, expected %s\n", __LINE__, #call, got_, #want);           \
            ++g_failed;                                                                           \
        }                                                                                         \
    }                                                                                             \
    while (0)
#define EXPECT_STR(want, call)                                                          \
    do                                                                                  \
    {                                                                                   \
        const char *got_ = (call);                                                      \
        if (strcmp(got_, want) != 0)                                                    \
        {                                                                               \
            printf("line %d: %s -> \"%s\", expected \"%s\"\n", __LINE__, #call, got_, want); \
            ++g_failed;                                                                 \
        }                                                                               \
    }                                                                                   \
    while (0)

#define BAD_ARG NVCV_ERROR_INVALID_ARGUMENT
#define OK NVCV_SUCCESS

static void *HeapAlloc(void *ctx, int64_t size, int32_t align)
{
    (void)ctx;
    void *p = NULL;
    return posix_memalign(&p, align < (int32_t)sizeof(void *) ? sizeof(void *) : (size_t)align, size ? (size_t)size : 1) == 0 ? p : NULL;
}

static void HeapFree(void *ctx, void *ptr, int64_t size, int32_t align)
{
    (void)ctx, (void)size, (void)align;
    free(ptr);
}

static void NoCleanup(void *ctx, NVCVResourceAllocator *a)
{
    (void)ctx, (void)a;
}

static NVCVResourceAllocator HeapResource(NVCVResourceType type)
{
    NVCVResourceAllocator r;
    memset(&r, 0, sizeof(r));
    r.resType         = type;
    r.res.mem.fnAlloc = HeapAlloc;
    r.res.mem.fnFree  = HeapFree;
    r.cleanup         = NoCleanup;
    return r;
}

static NVCVAllocatorHandle HeapAllocator(void)
{
    NVCVResourceAllocator res[3] = {HeapResource(NVCV_RESOURCE_MEM_HOST), HeapResource(NVCV_RESOURCE_MEM_CUDA),
                                    HeapResource(NVCV_RESOURCE_MEM_HOST_PINNED)};
    NVCVAllocatorHandle   h      = NULL;
    EXPECT(OK, nvcvAllocatorConstructCustom(res, 3, &h));
    return h;
}

static void TensorRequirementCases(void)
{
    NVCVTensorRequirements reqs;
    const NVCVImageFormat  rgba = NVCV_IMAGE_FORMAT_RGBA8;
    EXPECT(BAD_ARG, nvcvTensorCalcRequirementsForImages(-1, 224, 224, rgba, 0, 0, &reqs));
    EXPECT(BAD_ARG, nvcvTensorCalcRequirementsForImages(5, -1, 224, rgba, 0, 0, &reqs));
    EXPECT(BAD_ARG, nvcvTensorCalcRequirementsForImages(5, 224, -1, rgba, 0, 0, &reqs));
    EXPECT(BAD_ARG, nvcvTensorCalcRequirementsForImages(5, 224, 224, NVCV_IMAGE_FORMAT_NONE, 0, 0, &reqs));
    EXPECT(BAD_ARG, nvcvTensorCalcRequirementsForImages(5, 224, 224, rgba, 3, 0, &reqs));
    EXPECT(BAD_ARG, nvcvTensorCalcRequirementsForImages(5, 224, 224, rgba, 0, 3, &reqs));
    EXPECT(BAD_ARG, nvcvTensorCalcRequirementsForImages(5, 224, 224, rgba, 0, 0, NULL));
    /* block-linear memory and subsampled chroma cannot form a tensor ... */
    EXPECT(NVCV_ERROR_NOT_IMPLEMENTED,
           nvcvTensorCalcRequirementsForImages(
               5, 224, 224, NVCV_DETAIL_MAKE_COLOR_FMT1(RGB, UNDEFINED, BL, UNSIGNED, XYZW, ASSOCIATED, X8_Y8_Z8_W8), 0,
               0, &reqs));
    EXPECT(NVCV_ERROR_NOT_IMPLEMENTED,
           nvcvTensorCalcRequirementsForImages(5, 224, 224, NVCV_IMAGE_FORMAT_UYVY, 0, 0, &reqs));
    /* ... and planes must agree: semi-planar 4:4:4 and mixed plane depths are argument errors */
    EXPECT(BAD_ARG, nvcvTensorCalcRequirementsForImages(5, 224, 224, NVCV_IMAGE_FORMAT_NV24, 0, 0, &reqs));
    EXPECT(BAD_ARG,
           nvcvTensorCalcRequirementsForImages(
               5, 224, 224, NVCV_DETAIL_MAKE_COLOR_FMT4(RGB, UNDEFINED, PL, UNSIGNED, XYZW, ASSOCIATED, X8, X8, X8, X32),
               0, 0, &reqs));

    int64_t                wh[2] = {224, 224};
    const NVCVTensorLayout hw = NVCV_TENSOR_LAYOUT_MAKE("HW"), empty = NVCV_TENSOR_LAYOUT_MAKE("");
    EXPECT(BAD_ARG, nvcvTensorCalcRequirements(2, wh, NVCV_DATA_TYPE_NONE, hw, 0, 0, &reqs));
    EXPECT(BAD_ARG, nvcvTensorCalcRequirements(3, wh, NVCV_DATA_TYPE_U8, hw, 0, 0, &reqs));
    EXPECT(BAD_ARG, nvcvTensorCalcRequirements(-1, wh, NVCV_DATA_TYPE_U8, empty, 0, 0, &reqs));
    EXPECT(BAD_ARG, nvcvTensorCalcRequirements(2, wh, NVCV_DATA_TYPE_U8, NVCV_TENSOR_NONE, 3, 0, &reqs));
    EXPECT(BAD_ARG, nvcvTensorCalcRequirements(2, wh, NVCV_DATA_TYPE_U8, NVCV_TENSOR_NONE, 0, 3, &reqs));
    EXPECT(BAD_ARG, nvcvTensorCalcRequirements(2, wh, NVCV_DATA_TYPE_U8, NVCV_TENSOR_NONE, 0, 0, NULL));
}

static void TensorObjectCases(NVCVAllocatorHandle alloc)
{
    NVCVTensorRequirements reqs;
    NVCVTensorHandle       handle = NULL, other = NULL;
    EXPECT(OK, nvcvTensorCalcRequirementsForImages(1, 224, 224, NVCV_IMAGE_FORMAT_RGBA8, 0, 0, &reqs));
    EXPECT(BAD_ARG, nvcvTensorConstruct(NULL, alloc, &handle));
    EXPECT(BAD_ARG, nvcvTensorConstruct(&reqs, alloc, NULL));
    EXPECT(OK, nvcvTensorConstruct(&reqs, alloc, &handle));

    NVCVTensorData data;
    memset(&data, 0, sizeof(data));
    data.bufferType = NVCV_TENSOR_BUFFER_STRIDED_CUDA;
    data.layout     = NVCV_TENSOR_NHWC;
    data.rank       = 4;
    data.dtype      = NVCV_DATA_TYPE_F32;
    const int64_t shape[4] = {1, 224, 224, 3}, strides[4] = {224 * 224 * 12, 224 * 12, 12, 4};
    for (int i = 0; i < 4; ++i)
    {
        data.shape[i]                  = shape[i];
        data.buffer.strided.strides[i] = strides[i];
    }
    data.buffer.strided.basePtr = (NVCVByte *)0x1000;
    EXPECT(BAD_ARG, nvcvTensorWrapDataConstruct(NULL, NULL, NULL, &other));
    EXPECT(BAD_ARG, nvcvTensorWrapDataConstruct(&data, NULL, NULL, NULL));

    NVCVTensorLayout layout;
    EXPECT(BAD_ARG, nvcvTensorGetLayout(NULL, &layout));
    EXPECT(BAD_ARG, nvcvTensorGetLayout(handle, NULL));
    EXPECT(BAD_ARG, nvcvTensorExportData(NULL, &data));
    EXPECT(BAD_ARG, nvcvTensorExportData(handle, NULL));
    int32_t rank = NVCV_TENSOR_MAX_RANK;
    int64_t got[NVCV_TENSOR_MAX_RANK];
    EXPECT(BAD_ARG, nvcvTensorGetShape(NULL, &rank, got));
    EXPECT(BAD_ARG, nvcvTensorGetShape(handle, NULL, got));
    void *user;
    EXPECT(BAD_ARG, nvcvTensorGetUserPointer(NULL, &user));
    EXPECT(BAD_ARG, nvcvTensorGetUserPointer(handle, NULL));
    EXPECT(BAD_ARG, nvcvTensorGetAllocator(handle, NULL));
    EXPECT(BAD_ARG, nvcvTensorGetDataType(handle, NULL));

    int64_t chw[3] = {4, 224, 224};
    EXPECT(BAD_ARG, nvcvTensorReshape(NULL, 3, chw, NVCV_TENSOR_CHW, &other));
    EXPECT(BAD_ARG, nvcvTensorReshape(handle, 0, chw, NVCV_TENSOR_CHW, &other));
    EXPECT(BAD_ARG, nvcvTensorReshape(handle, NVCV_TENSOR_MAX_RANK + 1, chw, NVCV_TENSOR_CHW, &other));
    EXPECT(BAD_ARG, nvcvTensorReshape(handle, 3, chw, NVCV_TENSOR_HW, &other));
    EXPECT(BAD_ARG, nvcvTensorReshape(handle, 3, chw, NVCV_TENSOR_CHW, NULL));
    /* the same call with everything in place is a view of the one NHWC sample as 4 planes */
    EXPECT(OK, nvcvTensorReshape(handle, 3, chw, NVCV_TENSOR_CHW, &other));
    EXPECT(OK, nvcvTensorDecRef(other, NULL));
    {
        /* a unit dimension whose stride does not continue its neighbours: this build steps over it (no element of it
         * is ever addressed) and gives the 12 dense elements as one dimension; the reference's merge of contiguous
         * dimensions lets it split the run and refuses (src/nvcv/src/priv/TensorData.cpp:196-246) */
        NVCVTensorData odd;
        memset(&odd, 0, sizeof(odd));
        odd.bufferType = NVCV_TENSOR_BUFFER_STRIDED_CUDA;
        odd.rank       = 3;
        odd.dtype      = NVCV_DATA_TYPE_U8;
        EXPECT(OK, nvcvTensorLayoutMake("HWC", &odd.layout));
        const int64_t oshape[3] = {4, 1, 3}, ostrides[3] = {3, 999, 1};
        for (int i = 0; i < 3; ++i)
        {
            odd.shape[i]                  = oshape[i];
            odd.buffer.strided.strides[i] = ostrides[i];
        }
        odd.buffer.strided.basePtr = (NVCVByte *)0x2000;
        NVCVTensorHandle wrapped = NULL, flat = NULL;
        EXPECT(OK, nvcvTensorWrapDataConstruct(&odd, NULL, NULL, &wrapped));
        const int64_t    twelve[1] = {12};
        NVCVTensorLayout w;
        EXPECT(OK, nvcvTensorLayoutMake("W", &w));
        EXPECT(OK, nvcvTensorReshape(wrapped, 1, twelve, w, &flat));
        NVCVTensorData seen;
        EXPECT(OK, nvcvTensorExportData(flat, &seen));
        EXPECT(1, (int)seen.buffer.strided.strides[0]);
        EXPECT(OK, nvcvTensorDecRef(flat, NULL));
        EXPECT(OK, nvcvTensorDecRef(wrapped, NULL));
    }

    int newRef = -1;
    EXPECT(OK, nvcvTensorDecRef(handle, &newRef));
    EXPECT(0, newRef);
}

static void PermuteCases(void)
{
    int64_t src[5] = {16, 61, 23, 3, 0}, out[5];
    EXPECT(BAD_ARG, nvcvTensorShapePermute(NVCV_TENSOR_NHWC, NULL, NVCV_TENSOR_NCHW, out));
    EXPECT(BAD_ARG, nvcvTensorShapePermute(NVCV_TENSOR_NHWC, src, NVCV_TENSOR_NCHW, NULL));

    const struct
    {
        NVCVTensorLayout from, to;
        int              n;
        int64_t          in[5], gold[5];
    } rows[] = {
        { NVCV_TENSOR_NHWC,  NVCV_TENSOR_NCHW, 4,   {16, 61, 23, 3},   {16, 3, 61, 23}},
        {  NVCV_TENSOR_CHW,   NVCV_TENSOR_HWC, 3,       {3, 61, 23},       {61, 23, 3}},
        {NVCV_TENSOR_CFDHW, NVCV_TENSOR_FDHWC, 5, {3, 2, 6, 61, 23}, {2, 6, 61, 23, 3}},
        {  NVCV_TENSOR_CHW,    NVCV_TENSOR_HW, 2,       {3, 61, 23},          {61, 23}},
        {  NVCV_TENSOR_HWC,    NVCV_TENSOR_HW, 2,       {61, 23, 3},          {61, 23}},
    };
    for (size_t r = 0; r < sizeof(rows) / sizeof(rows[0]); ++r)
    {
        EXPECT(OK, nvcvTensorShapePermute(rows[r].from, rows[r].in, rows[r].to, out));
        EXPECT(0, memcmp(out, rows[r].gold, rows[r].n * sizeof(int64_t)));
    }
}

static NVCVImageHandle MakeImage(NVCVAllocatorHandle alloc, int w, int h, NVCVImageFormat fmt)
{
    NVCVImageRequirements reqs;
    NVCVImageHandle       img = NULL;
    EXPECT(OK, nvcvImageCalcRequirements(w, h, fmt, 0, 0, &reqs));
    EXPECT(OK, nvcvImageConstruct(&reqs, alloc, &img));
    return img;
}

/* What the tensor requirements, a tensor built from them and tensors wrapping data or an image look like. */
static int32_t g_lastDeviceAlign;

static void *RecordingAlloc(void *ctx, int64_t size, int32_t align)
{
    g_lastDeviceAlign = align;
    return HeapAlloc(ctx, size, align);
}

static int SameLayout(NVCVTensorLayout a, NVCVTensorLayout b)
{
    return a.rank == b.rank && memcmp(a.data, b.data, (size_t)a.rank) == 0;
}

static void TensorShapeCases(NVCVAllocatorHandle alloc)
{
    NVCVTensorRequirements reqs;
    /* a batch of images as one tensor: planar formats give NCHW, interleaved ones NHWC */
    EXPECT(OK, nvcvTensorCalcRequirementsForImages(53, 32, 16, NVCV_IMAGE_FORMAT_RGBA8p, 0, 0, &reqs));
    {
        const int64_t gold[4] = {53, 4, 16, 32};
        EXPECT(4, reqs.rank);
        EXPECT(0, memcmp(reqs.shape, gold, sizeof(gold)));
        EXPECT(1, SameLayout(reqs.layout, NVCV_TENSOR_NCHW));
        EXPECT(1, reqs.dtype == NVCV_DATA_TYPE_U8);
    }
    EXPECT(OK, nvcvTensorCalcRequirementsForImages(14, 64, 18, NVCV_IMAGE_FORMAT_RGB8, 0, 0, &reqs));
    {
        const int64_t gold[4] = {14, 18, 64, 3};
        EXPECT(4, reqs.rank);
        EXPECT(0, memcmp(reqs.shape, gold, sizeof(gold)));
        EXPECT(1, SameLayout(reqs.layout, NVCV_TENSOR_NHWC));
        EXPECT(1, reqs.dtype == NVCV_DATA_TYPE_U8);
    }

    /* rows padded to 32 bytes */
    const struct
    {
        NVCVTensorLayout layout;
        int              rank;
        int64_t          shape[4], strides[4];
    } rows[] = {
        {NVCV_TENSOR_NCHW, 4, {53, 4, 16, 17}, {4 * 16 * 32, 16 * 32, 32, 1}},
        {NVCV_TENSOR_NHWC, 4, {53, 17, 16, 3},         {17 * 64, 64, 3, 1}},
        { NVCV_TENSOR_CHW, 3,     {4, 16, 17},            {16 * 32, 32, 1}},
        { NVCV_TENSOR_HWC, 3,     {17, 16, 3},                  {64, 3, 1}},
    };
    for (size_t r = 0; r < sizeof(rows) / sizeof(rows[0]); ++r)
    {
        NVCVTensorHandle t = NULL;
        NVCVTensorData   d;
        EXPECT(OK, nvcvTensorCalcRequirements(rows[r].rank, rows[r].shape, NVCV_DATA_TYPE_U8, rows[r].layout, 0, 32, &reqs));
        EXPECT(0, memcmp(reqs.strides, rows[r].strides, rows[r].rank * sizeof(int64_t)));
        EXPECT(OK, nvcvTensorConstruct(&reqs, alloc, &t));
        EXPECT(OK, nvcvTensorExportData(t, &d));
        EXPECT(NVCV_TENSOR_BUFFER_STRIDED_CUDA, d.bufferType);
        EXPECT(rows[r].rank, d.rank);
        EXPECT(0, memcmp(d.shape, rows[r].shape, rows[r].rank * sizeof(int64_t)));
        EXPECT(0, memcmp(d.buffer.strided.strides, rows[r].strides, rows[r].rank * sizeof(int64_t)));
        EXPECT(1, d.buffer.strided.basePtr != NULL);
        EXPECT(OK, nvcvTensorDecRef(t, NULL));
    }

    /* packed rows, 32-byte base: the allocator is asked for exactly that alignment */
    NVCVResourceAllocator rec = HeapResource(NVCV_RESOURCE_MEM_CUDA);
    rec.res.mem.fnAlloc       = RecordingAlloc;
    NVCVAllocatorHandle recording = NULL;
    NVCVTensorHandle    t = NULL, wrapped = NULL;
    NVCVTensorData      d, w;
    EXPECT(OK, nvcvAllocatorConstructCustom(&rec, 1, &recording));
    EXPECT(OK, nvcvTensorCalcRequirementsForImages(5, 163, 117, NVCV_IMAGE_FORMAT_RGBA8, 32, 1, &reqs));
    g_lastDeviceAlign = 0;
    EXPECT(OK, nvcvTensorConstruct(&reqs, recording, &t));
    EXPECT(32, g_lastDeviceAlign);
    EXPECT(OK, nvcvTensorExportData(t, &d));
    EXPECT(1, d.buffer.strided.strides[3]);
    EXPECT(4, d.buffer.strided.strides[2]);
    EXPECT(163 * 4, d.buffer.strided.strides[1]);
    EXPECT(117 * 163 * 4, d.buffer.strided.strides[0]);
    NVCVAllocatorHandle got = NULL;
    EXPECT(OK, nvcvTensorGetAllocator(t, &got));
    EXPECT(1, got == recording);
    EXPECT(OK, nvcvAllocatorDecRef(got, NULL)); /* the getter hands out a reference */
    EXPECT(OK, nvcvTensorDecRef(t, NULL));
    EXPECT(OK, nvcvAllocatorDecRef(recording, NULL));

    /* two half-float planes: NCHW with two channels, and a tensor wrapping the exported data is its twin */
    NVCVImageFormat twoPlanes = NVCV_DETAIL_MAKE_COLOR_FMT2(RGB, BT601_ER, PL, FLOAT, XY00, ASSOCIATED, X16, X16);
    EXPECT(OK, nvcvTensorCalcRequirementsForImages(5, 173, 79, twoPlanes, 32, 1, &reqs));
    EXPECT(OK, nvcvTensorConstruct(&reqs, alloc, &t));
    EXPECT(OK, nvcvTensorExportData(t, &d));
    {
        const int64_t gold[4] = {5, 2, 79, 173};
        EXPECT(4, d.rank);
        EXPECT(0, memcmp(d.shape, gold, sizeof(gold)));
        EXPECT(1, SameLayout(d.layout, NVCV_TENSOR_NCHW));
        EXPECT(1, d.dtype == NVCV_DATA_TYPE_F16);
        EXPECT(2, d.buffer.strided.strides[3]);
        EXPECT(173 * 2, d.buffer.strided.strides[2]);
    }
    EXPECT(OK, nvcvTensorWrapDataConstruct(&d, NULL, NULL, &wrapped));
    EXPECT(OK, nvcvTensorExportData(wrapped, &w));
    EXPECT(d.rank, w.rank);
    EXPECT(0, memcmp(d.shape, w.shape, 4 * sizeof(int64_t)));
    EXPECT(0, memcmp(d.buffer.strided.strides, w.buffer.strided.strides, 4 * sizeof(int64_t)));
    EXPECT(1, SameLayout(d.layout, w.layout));
    EXPECT(1, d.dtype == w.dtype);
    EXPECT(1, d.buffer.strided.basePtr == w.buffer.strided.basePtr);
    got = alloc;
    EXPECT(OK, nvcvTensorGetAllocator(wrapped, &got));
    EXPECT(1, got == NULL); /* foreign memory: no allocator */
    EXPECT(OK, nvcvTensorDecRef(wrapped, NULL));
    EXPECT(OK, nvcvTensorDecRef(t, NULL));

    /* one image seen as a tensor */
    const struct
    {
        NVCVImageFormat  fmt;
        int64_t          shape[4];
        NVCVTensorLayout layout;
        NVCVDataType     dtype;
    } views[] = {
        {NVCV_IMAGE_FORMAT_RGBA8p, {1, 4, 23, 61}, NVCV_TENSOR_NCHW,  NVCV_DATA_TYPE_U8},
        { NVCV_IMAGE_FORMAT_RGBA8, {1, 23, 61, 4}, NVCV_TENSOR_NHWC,  NVCV_DATA_TYPE_U8},
        {  NVCV_IMAGE_FORMAT_RGB8, {1, 23, 61, 3}, NVCV_TENSOR_NHWC,  NVCV_DATA_TYPE_U8},
        { NVCV_IMAGE_FORMAT_RGB8p, {1, 3, 23, 61}, NVCV_TENSOR_NCHW,  NVCV_DATA_TYPE_U8},
        {   NVCV_IMAGE_FORMAT_F32, {1, 1, 23, 61}, NVCV_TENSOR_NCHW, NVCV_DATA_TYPE_F32},
        {  NVCV_IMAGE_FORMAT_2F32, {1, 23, 61, 2}, NVCV_TENSOR_NHWC, NVCV_DATA_TYPE_F32},
    };
    for (size_t v = 0; v < sizeof(views) / sizeof(views[0]); ++v)
    {
        NVCVImageHandle img = MakeImage(alloc, 61, 23, views[v].fmt);
        NVCVImageData   id;
        EXPECT(OK, nvcvImageExportData(img, &id));
        EXPECT(OK, nvcvTensorWrapImageConstruct(img, &t));
        EXPECT(OK, nvcvTensorExportData(t, &d));
        EXPECT(4, d.rank);
        EXPECT(0, memcmp(d.shape, views[v].shape, 4 * sizeof(int64_t)));
        EXPECT(1, SameLayout(d.layout, views[v].layout));
        EXPECT(1, d.dtype == views[v].dtype);
        EXPECT(1, d.buffer.strided.basePtr == id.buffer.strided.planes[0].basePtr);
        const int channelFirst = d.layout.data[1] == 'C';
        const int32_t planes   = id.buffer.strided.numPlanes;
        EXPECT(channelFirst ? (int)views[v].shape[1] : 1, planes);
        int32_t pixelBytes = 0;
        EXPECT(OK, nvcvImageFormatGetPlanePixelStrideBytes(views[v].fmt, 0, &pixelBytes));
        EXPECT(id.buffer.strided.planes[0].rowStride, d.buffer.strided.strides[channelFirst ? 2 : 1]);
        EXPECT(pixelBytes, d.buffer.strided.strides[channelFirst ? 3 : 2]);
        for (int32_t p = 1; p < planes; ++p)
        {
            EXPECT(1, id.buffer.strided.planes[p].basePtr == d.buffer.strided.basePtr + p * d.buffer.strided.strides[1]);
        }
        EXPECT(OK, nvcvTensorDecRef(t, NULL));
        EXPECT(OK, nvcvImageDecRef(img, NULL));
    }
}

static void TensorFromImageCases(NVCVAllocatorHandle alloc)
{
    NVCVTensorHandle t   = NULL;
    NVCVImageHandle  img = MakeImage(alloc, 24, 24, NVCV_IMAGE_FORMAT_UYVY);
    EXPECT(BAD_ARG, nvcvTensorWrapImageConstruct(img, &t));
    EXPECT(OK, nvcvImageDecRef(img, NULL));

    img = MakeImage(alloc, 24, 24, NVCV_DETAIL_MAKE_COLOR_FMT3(RGB, UNDEFINED, PL, UNSIGNED, XYZ0, ASSOCIATED, X8, X8, X16));
    EXPECT(BAD_ARG, nvcvTensorWrapImageConstruct(img, &t));
    EXPECT(OK, nvcvImageDecRef(img, NULL));

    img = MakeImage(alloc, 24, 24, NVCV_IMAGE_FORMAT_U8);
    EXPECT(BAD_ARG, nvcvTensorWrapImageConstruct(NULL, &t));
    EXPECT(BAD_ARG, nvcvTensorWrapImageConstruct(img, NULL));
    EXPECT(OK, nvcvImageDecRef(img, NULL));
}

static NVCVImageData OnePlane(NVCVImageFormat fmt, NVCVImageBufferType type)
{
    NVCVImageData d;
    memset(&d, 0, sizeof(d));
    d.format                             = fmt;
    d.bufferType                         = type;
    d.buffer.strided.numPlanes           = 1;
    d.buffer.strided.planes[0].width     = 173;
    d.buffer.strided.planes[0].height    = 79;
    d.buffer.strided.planes[0].rowStride = 190;
    d.buffer.strided.planes[0].basePtr   = (NVCVByte *)678;
    return d;
}

/* A fixed pool size caps the live objects of a kind: the next creation reports OUT_OF_MEMORY, a freed slot can be
 * taken again, and the size cannot be changed while objects are alive. Must run before anything else is created. */
enum Kind
{
    KIND_TENSOR,
    KIND_IMAGE,
    KIND_ALLOCATOR,
    KIND_BATCH /* needs a GPU */
};

static NVCVStatus Create(enum Kind kind, void **out)
{
    if (kind == KIND_TENSOR)
    {
        NVCVTensorData d;
        memset(&d, 0, sizeof(d));
        d.bufferType             = NVCV_TENSOR_BUFFER_STRIDED_CUDA;
        d.layout                 = NVCV_TENSOR_NONE;
        d.rank                   = 3;
        d.dtype                  = NVCV_DATA_TYPE_U8;
        const int64_t shape[3]   = {32, 12, 4};
        const int64_t strides[3] = {48, 4, 1};
        memcpy(d.shape, shape, sizeof(shape));
        memcpy(d.buffer.strided.strides, strides, sizeof(strides));
        d.buffer.strided.basePtr = (NVCVByte *)0x1000;
        return nvcvTensorWrapDataConstruct(&d, NULL, NULL, (NVCVTensorHandle *)out);
    }
    if (kind == KIND_IMAGE)
    {
        NVCVImageData d = OnePlane(NVCV_IMAGE_FORMAT_U8, NVCV_IMAGE_BUFFER_STRIDED_CUDA);
        return nvcvImageWrapDataConstruct(&d, NULL, NULL, (NVCVImageHandle *)out);
    }
    if (kind == KIND_BATCH)
    {
        NVCVImageBatchVarShapeRequirements reqs;
        NVCVStatus                         st = nvcvImageBatchVarShapeCalcRequirements(32, &reqs);
        return st != NVCV_SUCCESS ? st : nvcvImageBatchVarShapeConstruct(&reqs, NULL, (NVCVImageBatchHandle *)out);
    }
    return nvcvAllocatorConstructCustom(NULL, 0, (NVCVAllocatorHandle *)out);
}

static NVCVStatus Destroy(enum Kind kind, void *h)
{
    return kind == KIND_TENSOR  ? nvcvTensorDecRef((NVCVTensorHandle)h, NULL)
         : kind == KIND_IMAGE ? nvcvImageDecRef((NVCVImageHandle)h, NULL)
         : kind == KIND_BATCH ? nvcvImageBatchDecRef((NVCVImageBatchHandle)h, NULL)
                              : nvcvAllocatorDecRef((NVCVAllocatorHandle)h, NULL);
}

static NVCVStatus SetMax(enum Kind kind, int32_t n)
{
    return kind == KIND_TENSOR  ? nvcvConfigSetMaxTensorCount(n)
         : kind == KIND_IMAGE ? nvcvConfigSetMaxImageCount(n)
         : kind == KIND_BATCH ? nvcvConfigSetMaxImageBatchCount(n)
                              : nvcvConfigSetMaxAllocatorCount(n);
}

static void ConfigCases(int withBatches)
{
    for (int k = KIND_TENSOR; k <= (withBatches ? KIND_BATCH : KIND_ALLOCATOR); ++k)
    {
        enum Kind kind = (enum Kind)k;
        void     *objs[5], *extra = NULL;
        EXPECT(OK, SetMax(kind, 5));
        for (int i = 0; i < 5; ++i)
        {
            EXPECT(OK, Create(kind, &objs[i]));
        }
        EXPECT(NVCV_ERROR_OUT_OF_MEMORY, Create(kind, &extra));
        EXPECT(OK, Destroy(kind, objs[4]));
        EXPECT(OK, Create(kind, &objs[4]));
        EXPECT(NVCV_ERROR_OUT_OF_MEMORY, Create(kind, &extra));
        EXPECT(NVCV_ERROR_INVALID_OPERATION, SetMax(kind, 7));
        for (int i = 0; i < 5; ++i)
        {
            EXPECT(OK, Destroy(kind, objs[i]));
        }
        EXPECT(OK, SetMax(kind, 7));
        EXPECT(OK, SetMax(kind, -1)); /* back to pools that grow */
    }
    EXPECT(OK, nvcvConfigSetMaxArrayCount(3));
    EXPECT(OK, nvcvConfigSetMaxArrayCount(-1));
}

static void ImageCases(NVCVAllocatorHandle alloc)
{
    NVCVImageRequirements reqs;
    NVCVImageHandle       handle = NULL, wrapped = NULL;
    EXPECT(BAD_ARG, nvcvImageCalcRequirements(224, 224, NVCV_IMAGE_FORMAT_RGBA8, 0, 3, &reqs));
    EXPECT(BAD_ARG, nvcvImageCalcRequirements(224, 224, NVCV_IMAGE_FORMAT_RGBA8, 3, 0, &reqs));

    EXPECT(OK, nvcvImageCalcRequirements(224, 224, NVCV_IMAGE_FORMAT_U8_BL, 0, 0, &reqs));
    EXPECT(NVCV_ERROR_NOT_IMPLEMENTED, nvcvImageConstruct(&reqs, alloc, &handle));

    EXPECT(OK, nvcvImageCalcRequirements(224, 224, NVCV_IMAGE_FORMAT_U8, 0, 0, &reqs));
    EXPECT(BAD_ARG, nvcvImageConstruct(NULL, alloc, &handle));
    EXPECT(BAD_ARG, nvcvImageConstruct(&reqs, alloc, NULL));
    EXPECT(OK, nvcvImageConstruct(&reqs, alloc, &handle));

    int32_t         w, h;
    NVCVImageFormat fmt;
    NVCVTypeImage   type;
    EXPECT(BAD_ARG, nvcvImageGetSize(handle, NULL, &h));
    EXPECT(BAD_ARG, nvcvImageGetSize(handle, &w, NULL));
    EXPECT(BAD_ARG, nvcvImageGetFormat(handle, NULL));
    EXPECT(BAD_ARG, nvcvImageGetFormat(NULL, &fmt));
    EXPECT(BAD_ARG, nvcvImageGetType(handle, NULL));
    EXPECT(BAD_ARG, nvcvImageGetType(NULL, &type));
    EXPECT(BAD_ARG, nvcvImageExportData(handle, NULL));
    EXPECT(BAD_ARG, nvcvImageGetUserPointer(handle, NULL));
    EXPECT(BAD_ARG, nvcvImageGetAllocator(handle, NULL));

    /* an image wrapping foreign memory has no allocator */
    NVCVImageData       exported;
    NVCVAllocatorHandle got = alloc;
    EXPECT(OK, nvcvImageExportData(handle, &exported));
    EXPECT(OK, nvcvImageWrapDataConstruct(&exported, NULL, NULL, &wrapped));
    EXPECT(OK, nvcvImageGetAllocator(wrapped, &got));
    EXPECT(1, got == NULL);
    EXPECT(OK, nvcvImageGetType(wrapped, &type));
    EXPECT(NVCV_TYPE_IMAGE_WRAPDATA, type);
    EXPECT(OK, nvcvImageDecRef(wrapped, NULL));
    EXPECT(OK, nvcvImageDecRef(handle, NULL));

    NVCVImageData d = OnePlane(NVCV_IMAGE_FORMAT_U8_BL, NVCV_IMAGE_BUFFER_STRIDED_CUDA);
    EXPECT(BAD_ARG, nvcvImageWrapDataConstruct(&d, NULL, NULL, &wrapped)); /* block-linear */
    d                          = OnePlane(NVCV_IMAGE_FORMAT_U8, NVCV_IMAGE_BUFFER_STRIDED_CUDA);
    d.buffer.strided.numPlanes = 0;
    EXPECT(BAD_ARG, nvcvImageWrapDataConstruct(&d, NULL, NULL, &wrapped)); /* format has one plane, buffer none */
    d = OnePlane(NVCV_IMAGE_FORMAT_U8, NVCV_IMAGE_BUFFER_STRIDED_CUDA);
    EXPECT(BAD_ARG, nvcvImageWrapDataConstruct(&d, NULL, NULL, NULL));
    EXPECT(BAD_ARG, nvcvImageWrapDataConstruct(NULL, NULL, NULL, &wrapped));
    d.buffer.strided.planes[0].basePtr = NULL;
    EXPECT(BAD_ARG, nvcvImageWrapDataConstruct(&d, NULL, NULL, &wrapped));
    /* only pitch-linear device memory can be wrapped */
    d = OnePlane(NVCV_IMAGE_FORMAT_U8, NVCV_IMAGE_BUFFER_CUDA_ARRAY);
    EXPECT(BAD_ARG, nvcvImageWrapDataConstruct(&d, NULL, NULL, &wrapped));
    d = OnePlane(NVCV_IMAGE_FORMAT_U8, NVCV_IMAGE_BUFFER_STRIDED_HOST);
    EXPECT(BAD_ARG, nvcvImageWrapDataConstruct(&d, NULL, NULL, &wrapped));
    d = OnePlane(NVCV_IMAGE_FORMAT_NONE, NVCV_IMAGE_BUFFER_NONE);
    EXPECT(BAD_ARG, nvcvImageWrapDataConstruct(&d, NULL, NULL, &wrapped));
}

static void AllocatorCases(void)
{
    NVCVResourceAllocator two[2] = {HeapResource(NVCV_RESOURCE_MEM_HOST), HeapResource(NVCV_RESOURCE_MEM_CUDA)};
    NVCVAllocatorHandle   h      = NULL;
    EXPECT(BAD_ARG, nvcvAllocatorConstructCustom(two, 2, NULL));
    EXPECT(OK, nvcvAllocatorConstructCustom(two, 2, &h));
    EXPECT(BAD_ARG, nvcvAllocatorGetUserPointer(h, NULL));
    EXPECT(BAD_ARG, nvcvAllocatorAllocHostMemory(h, NULL, 1 << 10, 256));
    EXPECT(BAD_ARG, nvcvAllocatorAllocHostPinnedMemory(h, NULL, 1 << 10, 256));
    EXPECT(BAD_ARG, nvcvAllocatorAllocCudaMemory(h, NULL, 1 << 10, 256));
    void *p = NULL;
    /* negative size, alignment not a power of two, size not a multiple of the alignment */
    EXPECT(BAD_ARG, nvcvAllocatorAllocHostMemory(h, &p, -1, 256));
    EXPECT(BAD_ARG, nvcvAllocatorAllocHostMemory(h, &p, 1 << 10, 3));
    EXPECT(BAD_ARG, nvcvAllocatorAllocHostMemory(h, &p, 128, 256));
    EXPECT(BAD_ARG, nvcvAllocatorAllocHostPinnedMemory(h, &p, -1, 256));
    EXPECT(BAD_ARG, nvcvAllocatorAllocHostPinnedMemory(h, &p, 1 << 10, 3));
    EXPECT(BAD_ARG, nvcvAllocatorAllocHostPinnedMemory(h, &p, 128, 256));
    EXPECT(BAD_ARG, nvcvAllocatorAllocCudaMemory(h, &p, -1, 256));
    EXPECT(BAD_ARG, nvcvAllocatorAllocCudaMemory(h, &p, 1 << 10, 3));
    EXPECT(BAD_ARG, nvcvAllocatorAllocCudaMemory(h, &p, 128, 256));
    EXPECT(OK, nvcvAllocatorAllocHostMemory(h, &p, 1 << 10, 256));
    EXPECT(0, (long long)((uintptr_t)p % 256));
    EXPECT(OK, nvcvAllocatorFreeHostMemory(h, p, 1 << 10, 256));
    int newRef = 1;
    EXPECT(OK, nvcvAllocatorDecRef(h, &newRef));
    EXPECT(0, newRef);

    NVCVResourceAllocator r = HeapResource(NVCV_RESOURCE_MEM_HOST);
    r.res.mem.fnAlloc       = NULL;
    EXPECT(BAD_ARG, nvcvAllocatorConstructCustom(&r, 1, &h));
    r                = HeapResource(NVCV_RESOURCE_MEM_CUDA);
    r.res.mem.fnFree = NULL;
    EXPECT(BAD_ARG, nvcvAllocatorConstructCustom(&r, 1, &h));
    NVCVResourceAllocator twice[2] = {HeapResource(NVCV_RESOURCE_MEM_HOST), HeapResource(NVCV_RESOURCE_MEM_HOST)};
    EXPECT(BAD_ARG, nvcvAllocatorConstructCustom(twice, 2, &h));

    EXPECT_STR("NVCV_RESOURCE_MEM_CUDA", nvcvResourceTypeGetName(NVCV_RESOURCE_MEM_CUDA));
    EXPECT_STR("NVCV_RESOURCE_MEM_HOST", nvcvResourceTypeGetName(NVCV_RESOURCE_MEM_HOST));
    EXPECT_STR("NVCV_RESOURCE_MEM_HOST_PINNED", nvcvResourceTypeGetName(NVCV_RESOURCE_MEM_HOST_PINNED));
    EXPECT_STR("Unexpected error retrieving NVCVResourceType string representation",
               nvcvResourceTypeGetName((NVCVResourceType)255));
}

/* Custom resources count their calls in their context: +1 per allocation, +10 per release; the cleanup callback
 * sees the final count and the stored descriptor. */
static void *CountingAlloc(void *ctx, int64_t size, int32_t align)
{
    *(int *)ctx += 1;
    return HeapAlloc(NULL, size, align);
}

static void CountingFree(void *ctx, void *ptr, int64_t size, int32_t align)
{
    *(int *)ctx += 10;
    HeapFree(NULL, ptr, size, align);
}

static void CountingCleanup(void *ctx, NVCVResourceAllocator *a)
{
    EXPECT(1, ctx == a->ctx);
    EXPECT(11, *(int *)ctx % 100);
    *(int *)ctx = -*(int *)ctx;
}

static void AllocatorUseCases(int device)
{
    int                   ctx[2] = {100, 200};
    NVCVResourceAllocator res[2];
    for (int i = 0; i < 2; ++i)
    {
        memset(&res[i], 0, sizeof(res[i]));
        res[i].resType         = i == 0 ? NVCV_RESOURCE_MEM_HOST : NVCV_RESOURCE_MEM_CUDA;
        res[i].ctx             = &ctx[i];
        res[i].res.mem.fnAlloc = CountingAlloc;
        res[i].res.mem.fnFree  = CountingFree;
        res[i].cleanup         = CountingCleanup;
    }
    NVCVAllocatorHandle h = NULL;
    EXPECT(OK, nvcvAllocatorConstructCustom(res, 2, &h));
    int refs = 0;
    EXPECT(OK, nvcvAllocatorRefCount(h, &refs));
    EXPECT(1, refs);
    for (int i = 0; i < 2; ++i)
    {
        NVCVResourceAllocator got;
        memset(&got, 0, sizeof(got));
        EXPECT(OK, nvcvAllocatorGet(h, res[i].resType, &got));
        EXPECT(res[i].resType, got.resType);
        EXPECT(1, got.ctx == res[i].ctx);
        EXPECT(1, got.res.mem.fnAlloc == res[i].res.mem.fnAlloc);
        EXPECT(1, got.res.mem.fnFree == res[i].res.mem.fnFree);
    }
    NVCVResourceAllocator pinned;
    EXPECT(OK, nvcvAllocatorGet(h, NVCV_RESOURCE_MEM_HOST_PINNED, &pinned)); /* the default one fills the gap */
    EXPECT(NVCV_RESOURCE_MEM_HOST_PINNED, pinned.resType);
    EXPECT(1, pinned.res.mem.fnAlloc != NULL && pinned.res.mem.fnFree != NULL);
    EXPECT(BAD_ARG, nvcvAllocatorGet(h, NVCV_RESOURCE_MEM_HOST, NULL));

    void *p = NULL;
    EXPECT(OK, nvcvAllocatorAllocHostMemory(h, &p, 1 << 20, 256));
    EXPECT(1, p != NULL);
    EXPECT(101, ctx[0]);
    EXPECT(OK, nvcvAllocatorFreeHostMemory(h, p, 1 << 20, 256));
    EXPECT(111, ctx[0]);
    EXPECT(OK, nvcvAllocatorAllocCudaMemory(h, &p, 1 << 20, 256));
    EXPECT(1, p != NULL);
    EXPECT(201, ctx[1]);
    EXPECT(OK, nvcvAllocatorFreeCudaMemory(h, p, 1 << 20, 256));
    EXPECT(211, ctx[1]);
    if (device)
    {
        p = NULL;
        EXPECT(OK, nvcvAllocatorAllocHostPinnedMemory(h, &p, 1 << 20, 256));
        EXPECT(1, p != NULL);
        EXPECT(OK, nvcvAllocatorFreeHostPinnedMemory(h, p, 1 << 20, 256));
    }

    void *user = (void *)1;
    EXPECT(OK, nvcvAllocatorGetUserPointer(h, &user));
    EXPECT(1, user == NULL);
    EXPECT(OK, nvcvAllocatorSetUserPointer(h, (void *)0x123));
    EXPECT(OK, nvcvAllocatorGetUserPointer(h, &user));
    EXPECT(1, user == (void *)0x123);
    EXPECT(OK, nvcvAllocatorSetUserPointer(h, NULL));
    EXPECT(OK, nvcvAllocatorGetUserPointer(h, &user));
    EXPECT(1, user == NULL);

    EXPECT(OK, nvcvAllocatorIncRef(h, &refs));
    EXPECT(2, refs);
    EXPECT(OK, nvcvAllocatorDecRef(h, &refs));
    EXPECT(1, refs);
    EXPECT(111, ctx[0]); /* not cleaned up while a reference is left */
    EXPECT(OK, nvcvAllocatorDecRef(h, &refs));
    EXPECT(0, refs);
    EXPECT(-111, ctx[0]);
    EXPECT(-211, ctx[1]);
}

#define BATCH_CAPACITY 32

static NVCVImageHandle g_pushed[BATCH_CAPACITY + 8];
static int             g_numPushed;
static int             g_pushLimit;

static NVCVImageHandle PushNext(void *ctx)
{
    NVCVAllocatorHandle alloc = (NVCVAllocatorHandle)ctx;
    if (g_numPushed >= g_pushLimit)
    {
        return NULL;
    }
    NVCVImageHandle img = MakeImage(alloc, 320 + g_numPushed * 2, 122 - g_numPushed * 2, NVCV_IMAGE_FORMAT_NV12);
    g_pushed[g_numPushed++] = img;
    return img; /* the batch takes over this reference */
}

static void ImageBatchCases(NVCVAllocatorHandle alloc)
{
    NVCVImageBatchVarShapeRequirements reqs;
    NVCVImageBatchHandle               batch = NULL;
    EXPECT(BAD_ARG, nvcvImageBatchVarShapeCalcRequirements(5, NULL));
    EXPECT(BAD_ARG, nvcvImageBatchVarShapeCalcRequirements(-1, &reqs));
    EXPECT(OK, nvcvImageBatchVarShapeCalcRequirements(BATCH_CAPACITY, &reqs));
    EXPECT(BAD_ARG, nvcvImageBatchVarShapeConstruct(NULL, NULL, &batch));
    EXPECT(BAD_ARG, nvcvImageBatchVarShapeConstruct(&reqs, NULL, NULL));
    EXPECT(OK, nvcvImageBatchVarShapeConstruct(&reqs, NULL, &batch));

    NVCVAllocatorHandle got = alloc;
    EXPECT(OK, nvcvImageBatchGetAllocator(batch, &got));
    EXPECT(1, got == NULL); /* built on the default allocator */
    EXPECT(BAD_ARG, nvcvImageBatchGetAllocator(batch, NULL));
    EXPECT(BAD_ARG, nvcvImageBatchGetUserPointer(batch, NULL));
    EXPECT(BAD_ARG, nvcvImageBatchGetNumImages(batch, NULL));
    EXPECT(BAD_ARG, nvcvImageBatchGetCapacity(batch, NULL));
    EXPECT(BAD_ARG, nvcvImageBatchVarShapeGetUniqueFormat(batch, NULL));
    EXPECT(BAD_ARG, nvcvImageBatchGetType(batch, NULL));
    EXPECT(BAD_ARG, nvcvImageBatchExportData(batch, 0, NULL));
    EXPECT(BAD_ARG, nvcvImageBatchVarShapeGetMaxSize(batch, NULL, NULL));

    NVCVImageHandle images[BATCH_CAPACITY + 1], out[BATCH_CAPACITY + 1];
    for (int i = 0; i < BATCH_CAPACITY + 1; ++i)
    {
        images[i] = MakeImage(alloc, 2 + 2 * (i % 4), 2 + 2 * ((i / 4) % 4), NVCV_IMAGE_FORMAT_NV12);
    }
    EXPECT(NVCV_ERROR_OVERFLOW, nvcvImageBatchVarShapePushImages(batch, images, BATCH_CAPACITY + 1));
    EXPECT(BAD_ARG, nvcvImageBatchVarShapePushImages(batch, NULL, BATCH_CAPACITY));
    int32_t n = -1;
    EXPECT(OK, nvcvImageBatchGetNumImages(batch, &n));
    EXPECT(0, n); /* a rejected push adds nothing */

    EXPECT(OK, nvcvImageBatchVarShapePushImages(batch, images, BATCH_CAPACITY));
    EXPECT(BAD_ARG, nvcvImageBatchVarShapePopImages(batch, -1));
    EXPECT(BAD_ARG, nvcvImageBatchVarShapeGetImages(batch, 0, NULL, BATCH_CAPACITY));
    EXPECT(BAD_ARG, nvcvImageBatchVarShapeGetImages(batch, -1, out, BATCH_CAPACITY));
    EXPECT(NVCV_ERROR_OVERFLOW, nvcvImageBatchVarShapeGetImages(batch, 0, out, BATCH_CAPACITY + 1));
    EXPECT(NVCV_ERROR_OVERFLOW, nvcvImageBatchVarShapeGetImages(batch, 1, out, BATCH_CAPACITY));
    EXPECT(OK, nvcvImageBatchVarShapeGetImages(batch, 0, out, BATCH_CAPACITY));
    EXPECT(0, memcmp(out, images, BATCH_CAPACITY * sizeof(images[0])));
    for (int i = 0; i < BATCH_CAPACITY; ++i)
    {
        EXPECT(OK, nvcvImageDecRef(out[i], NULL)); /* each handle handed out carries a reference */
    }
    EXPECT(OK, nvcvImageBatchVarShapePopImages(batch, BATCH_CAPACITY));
    EXPECT(NVCV_ERROR_UNDERFLOW, nvcvImageBatchVarShapePopImages(batch, 1));

    /* a producer that never stops overflows the batch; a missing producer is an argument error */
    g_numPushed = 0;
    g_pushLimit = BATCH_CAPACITY + 1;
    EXPECT(NVCV_ERROR_OVERFLOW, nvcvImageBatchVarShapePushImagesCallback(batch, PushNext, alloc));
    for (int i = 0; i < g_numPushed; ++i)
    {
        int newRef = -1;
        EXPECT(OK, nvcvImageDecRef(g_pushed[i], &newRef));
        EXPECT(0, newRef); /* nothing stayed in the batch */
    }
    EXPECT(BAD_ARG, nvcvImageBatchVarShapePushImagesCallback(batch, NULL, alloc));

    EXPECT(OK, nvcvImageBatchDecRef(batch, NULL));
    for (int i = 0; i < BATCH_CAPACITY + 1; ++i)
    {
        int newRef = -1;
        EXPECT(OK, nvcvImageDecRef(images[i], &newRef));
        EXPECT(0, newRef);
    }
}

int main(int argc, char **argv)
{
    const int device = argc > 1 && strcmp(argv[1], "device") == 0;
    ConfigCases(device);
    NVCVAllocatorHandle alloc = HeapAllocator();
    TensorRequirementCases();
    TensorObjectCases(alloc);
    PermuteCases();
    TensorShapeCases(alloc);
    TensorFromImageCases(alloc);
    ImageCases(alloc);
    AllocatorCases();
    AllocatorUseCases(device);
    if (device)
    {
        ImageBatchCases(alloc);
    }
    int newRef = -1;
    EXPECT(OK, nvcvAllocatorDecRef(alloc, &newRef));
    EXPECT(0, newRef);
    ConfigCases(device); /* once more, on pools that have grown meanwhile: nothing may be left alive, the caps hold */
    printf("%d failed\n", g_failed);
    return g_failed > 100 ? 100 : g_failed;
}
