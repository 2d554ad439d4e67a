/* Handles under concurrency, plain C with pthreads against the public headers (the reference exercises the same
 * machinery in tests/nvcv_types/unit/TestHandleManager.cpp and TestLockFreeStack.cpp through its private classes):
 *   - every thread creates, shares, queries and destroys tensors and images that wrap a fake device address, and
 *     tensors whose memory comes from one custom allocator that all threads share;
 *   - one object is shared by all threads through its reference count;
 *   - threads hand each other tensors through shared slots, each with a reference of its own, so that the last
 *     reference is dropped by whichever thread comes last;
 *   - every thread sets and reads back its own status message between calls that fail;
 *   - afterwards every wrapped tensor has run its cleanup exactly once, nothing is alive (the pools accept a fixed
 *     size) and a destroyed handle is refused through 15 reuses of its slot.
 * Usage: handle_pool_stress [threads [rounds]]; prints failures, exits with their count. */
#include <nvcv/alloc/Allocator.h>
#include <nvcv/Config.h>
#include <nvcv/Image.h>
#include <nvcv/Status.h>
#include <nvcv/Tensor.h>
#include <pthread.h>
#include <stdatomic.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static atomic_int g_failed;
static int        g_rounds = 4000;

#define CHECK(cond)                                                  \
    do                                                               \
    {                                                                \
        if (!(cond))                                                 \
        {                                                            \
            if (atomic_fetch_add(&g_failed, 1) < 20)                 \
            {                                                        \
                printf("line %d: %s\n", __LINE__, #cond);            \
            }                                                        \
        }                                                            \
    }                                                                \
    while (0)

static NVCVTensorData TensorOf(int rows)
{
    NVCVTensorData d;
    memset(&d, 0, sizeof(d));
    d.bufferType                = NVCV_TENSOR_BUFFER_STRIDED_CUDA;
    d.layout                    = NVCV_TENSOR_HWC;
    d.rank                      = 3;
    d.dtype                     = NVCV_DATA_TYPE_U8;
    d.shape[0]                  = rows;
    d.shape[1]                  = 8;
    d.shape[2]                  = 3;
    d.buffer.strided.strides[0] = 24;
    d.buffer.strided.strides[1] = 3;
    d.buffer.strided.strides[2] = 1;
    d.buffer.strided.basePtr    = (NVCVByte *)0x10000;
    return d;
}

static NVCVImageData ImageOf(int width)
{
    NVCVImageData d;
    memset(&d, 0, sizeof(d));
    d.format                             = NVCV_IMAGE_FORMAT_U8;
    d.bufferType                         = NVCV_IMAGE_BUFFER_STRIDED_CUDA;
    d.buffer.strided.numPlanes           = 1;
    d.buffer.strided.planes[0].width     = width;
    d.buffer.strided.planes[0].height    = 4;
    d.buffer.strided.planes[0].rowStride = 256;
    d.buffer.strided.planes[0].basePtr   = (NVCVByte *)0x20000;
    return d;
}

/* an object every thread holds a reference to for a while */
static NVCVTensorHandle g_shared;
/* slots through which threads hand each other tensors */
#define SLOTS 64
static _Atomic(NVCVTensorHandle) g_passed[SLOTS];
static atomic_int g_cleanups;

/* "device" memory from the host heap, counted: the library never touches what a tensor's buffer holds */
static atomic_long g_allocs, g_frees, g_allocatorCleanups;

static void *HeapAlloc(void *ctx, int64_t size, int32_t align)
{
    (void)ctx;
    void *p = NULL;
    atomic_fetch_add(&g_allocs, 1);
    return posix_memalign(&p, (size_t)align < sizeof(void *) ? sizeof(void *) : (size_t)align, size ? (size_t)size : 1) == 0
             ? p
             : NULL;
}

static void HeapFree(void *ctx, void *ptr, int64_t size, int32_t align)
{
    (void)ctx, (void)size, (void)align;
    atomic_fetch_add(&g_frees, 1);
    free(ptr);
}

static void AllocatorCleanup(void *ctx, NVCVResourceAllocator *a)
{
    (void)ctx, (void)a;
    atomic_fetch_add(&g_allocatorCleanups, 1);
}

static NVCVAllocatorHandle g_allocator;

static void CountCleanup(void *ctx, const NVCVTensorData *data)
{
    (void)ctx, (void)data;
    atomic_fetch_add(&g_cleanups, 1);
}

static void *Worker(void *arg)
{
    const int id = (int)(intptr_t)arg;
    unsigned  rnd = 12345u + 977u * (unsigned)id;
    int       created = 0;
    for (int r = 0; r < g_rounds; ++r)
    {
        rnd = rnd * 1664525u + 1013904223u;
        /* own objects: create, use, destroy */
        NVCVTensorData   td = TensorOf(1 + (int)(rnd >> 8) % 50);
        NVCVTensorHandle t  = NULL;
        CHECK(nvcvTensorWrapDataConstruct(&td, CountCleanup, NULL, &t) == NVCV_SUCCESS);
        ++created;
        int     rank = 3, refs = 0;
        int64_t shape[3];
        CHECK(nvcvTensorGetShape(t, &rank, shape) == NVCV_SUCCESS && shape[0] == td.shape[0]);
        CHECK(nvcvTensorIncRef(t, &refs) == NVCV_SUCCESS && refs == 2);
        CHECK(nvcvTensorDecRef(t, &refs) == NVCV_SUCCESS && refs == 1);
        NVCVImageData   id_ = ImageOf(1 + (int)(rnd >> 16) % 60);
        NVCVImageHandle img = NULL;
        CHECK(nvcvImageWrapDataConstruct(&id_, NULL, NULL, &img) == NVCV_SUCCESS);
        int32_t w = 0, h = 0;
        CHECK(nvcvImageGetSize(img, &w, &h) == NVCV_SUCCESS && w == id_.buffer.strided.planes[0].width && h == 4);
        /* a tensor handle is not an image handle, whichever thread made it */
        CHECK(nvcvImageGetSize((NVCVImageHandle)t, &w, &h) == NVCV_ERROR_INVALID_ARGUMENT);
        /* the status of the last call belongs to the calling thread (reference: tests/nvcv_types/system/
         * TestStatus.cpp, the thread-local status) */
        if (r % 16 == 0)
        {
            char want[NVCV_MAX_STATUS_MESSAGE_LENGTH], got[NVCV_MAX_STATUS_MESSAGE_LENGTH];
            snprintf(want, sizeof(want), "thread %d round %d", id, r);
            nvcvSetThreadStatus(NVCV_ERROR_INTERNAL, "thread %d round %d", id, r);
            CHECK(nvcvPeekAtLastErrorMessage(got, (int32_t)sizeof(got)) == NVCV_ERROR_INTERNAL && strcmp(got, want) == 0);
            CHECK(nvcvImageGetSize((NVCVImageHandle)t, &w, &h) == NVCV_ERROR_INVALID_ARGUMENT);
            CHECK(nvcvGetLastError() == NVCV_ERROR_INVALID_ARGUMENT); /* the failed call's, and that resets it */
            CHECK(nvcvGetLastError() == NVCV_SUCCESS);
        }
        CHECK(nvcvImageDecRef(img, &refs) == NVCV_SUCCESS && refs == 0);
        /* a tensor with memory of its own from the shared allocator, which it holds a reference to */
        if (r % 4 == 0)
        {
            NVCVTensorRequirements reqs;
            const int64_t          shp[3] = {1 + (int)(rnd >> 20) % 9, 16, 3};
            NVCVTensorHandle       owned  = NULL;
            CHECK(nvcvTensorCalcRequirements(3, shp, NVCV_DATA_TYPE_U8, NVCV_TENSOR_HWC, 0, 0, &reqs) == NVCV_SUCCESS);
            CHECK(nvcvTensorConstruct(&reqs, g_allocator, &owned) == NVCV_SUCCESS);
            NVCVTensorData od;
            CHECK(nvcvTensorExportData(owned, &od) == NVCV_SUCCESS && od.buffer.strided.basePtr != NULL
                  && od.shape[0] == shp[0]);
            CHECK(nvcvAllocatorRefCount(g_allocator, &refs) == NVCV_SUCCESS && refs >= 2);
            CHECK(nvcvTensorDecRef(owned, &refs) == NVCV_SUCCESS && refs == 0);
        }
        /* the shared object: one more reference for a while */
        CHECK(nvcvTensorIncRef(g_shared, &refs) == NVCV_SUCCESS && refs >= 2);
        /* hand the own tensor, with a reference of its own, to whoever looks at the slot next, and take over what
         * lies there together with its reference */
        const int slot = (int)(rnd >> 4) % SLOTS;
        CHECK(nvcvTensorIncRef(t, &refs) == NVCV_SUCCESS && refs == 2);
        NVCVTensorHandle other = atomic_exchange(&g_passed[slot], t);
        if (other != NULL)
        {
            rank = 3;
            CHECK(nvcvTensorGetShape(other, &rank, shape) == NVCV_SUCCESS && shape[1] == 8 && shape[2] == 3);
            CHECK(nvcvTensorRefCount(other, &refs) == NVCV_SUCCESS && refs >= 1 && refs <= 2);
            CHECK(nvcvTensorDecRef(other, &refs) == NVCV_SUCCESS && refs >= 0 && refs <= 1);
        }
        CHECK(nvcvTensorDecRef(g_shared, &refs) == NVCV_SUCCESS && refs >= 1);
        CHECK(nvcvTensorDecRef(t, &refs) == NVCV_SUCCESS && refs >= 0 && refs <= 1);
        /* the image is gone: its handle is refused, unless 16 later objects have used the slot by now and the
         * 4-bit generation has come round */
        NVCVStatus st = nvcvImageRefCount(img, &refs);
        CHECK(st == NVCV_ERROR_INVALID_ARGUMENT || st == NVCV_SUCCESS);
    }
    return (void *)(intptr_t)created;
}

int main(int argc, char **argv)
{
    int threads = argc > 1 ? atoi(argv[1]) : 8;
    if (argc > 2)
    {
        g_rounds = atoi(argv[2]);
    }
    if (threads < 1 || threads > 64)
    {
        threads = 8;
    }
    NVCVResourceAllocator res;
    memset(&res, 0, sizeof(res));
    res.resType         = NVCV_RESOURCE_MEM_CUDA;
    res.res.mem.fnAlloc = HeapAlloc;
    res.res.mem.fnFree  = HeapFree;
    res.cleanup         = AllocatorCleanup;
    CHECK(nvcvAllocatorConstructCustom(&res, 1, &g_allocator) == NVCV_SUCCESS);
    NVCVTensorData shared = TensorOf(7);
    CHECK(nvcvTensorWrapDataConstruct(&shared, NULL, NULL, &g_shared) == NVCV_SUCCESS);
    pthread_t th[64];
    for (int i = 0; i < threads; ++i)
    {
        CHECK(pthread_create(&th[i], NULL, Worker, (void *)(intptr_t)i) == 0);
    }
    long created = 0;
    for (int i = 0; i < threads; ++i)
    {
        void *ret = NULL;
        CHECK(pthread_join(th[i], &ret) == 0);
        created += (long)(intptr_t)ret;
    }
    int refs = -1;
    for (int i = 0; i < SLOTS; ++i)
    {
        NVCVTensorHandle left = atomic_exchange(&g_passed[i], NULL);
        if (left != NULL)
        {
            CHECK(nvcvTensorDecRef(left, &refs) == NVCV_SUCCESS && refs == 0);
        }
    }
    CHECK(nvcvTensorRefCount(g_shared, &refs) == NVCV_SUCCESS && refs == 1);
    CHECK(nvcvTensorDecRef(g_shared, &refs) == NVCV_SUCCESS && refs == 0);
    CHECK(atomic_load(&g_cleanups) == created); /* every wrapped tensor ran its cleanup exactly once */
    CHECK(nvcvAllocatorRefCount(g_allocator, &refs) == NVCV_SUCCESS && refs == 1); /* no tensor holds it any more */
    CHECK(nvcvAllocatorDecRef(g_allocator, &refs) == NVCV_SUCCESS && refs == 0);
    CHECK(atomic_load(&g_allocs) == atomic_load(&g_frees) && atomic_load(&g_allocs) > 0);
    CHECK(atomic_load(&g_allocatorCleanups) == 1);
    /* a destroyed handle stays refused while later objects take its slot */
    CHECK(nvcvConfigSetMaxTensorCount(1) == NVCV_SUCCESS); /* one slot in use from here on */
    NVCVTensorHandle gone = NULL;
    CHECK(nvcvTensorWrapDataConstruct(&shared, NULL, NULL, &gone) == NVCV_SUCCESS);
    CHECK(nvcvTensorDecRef(gone, NULL) == NVCV_SUCCESS);
    for (int i = 0; i < 15; ++i)
    {
        NVCVTensorHandle next = NULL;
        CHECK(nvcvTensorWrapDataConstruct(&shared, NULL, NULL, &next) == NVCV_SUCCESS);
        CHECK(next != gone);
        CHECK(nvcvTensorRefCount(gone, &refs) == NVCV_ERROR_INVALID_ARGUMENT);
        CHECK(nvcvTensorDecRef(next, NULL) == NVCV_SUCCESS);
    }
    /* nothing is alive: the pools accept a fixed size */
    CHECK(nvcvConfigSetMaxTensorCount(3) == NVCV_SUCCESS);
    CHECK(nvcvConfigSetMaxImageCount(3) == NVCV_SUCCESS);
    CHECK(nvcvConfigSetMaxTensorCount(-1) == NVCV_SUCCESS);
    CHECK(nvcvConfigSetMaxImageCount(-1) == NVCV_SUCCESS);
    printf("%d threads x %d rounds, %ld tensors: %d failed\n", threads, g_rounds, created, atomic_load(&g_failed));
    return atomic_load(&g_failed) > 100 ? 100 : atomic_load(&g_failed);
}
