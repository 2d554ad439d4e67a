// Variable-shape image batch: host-side descriptor arrays mirrored in device memory.
// Behaviour follows src/nvcv/src/priv/ImageBatchVarShape.cpp:38-430 of the reference. Differences by
// design: the host mirror lives in pinned memory so the upload issued by exportData() is a true
// asynchronous DMA on the caller's stream, and the host mirror can be read by operators to pack
// their launch grids (nvcvxImageBatchVarShapeGetHostImageList).
#include "Priv.hpp"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <numeric>

namespace nvcvamd {

namespace {

void CheckHip(hipError_t e, const char *what)
{
    if (e != hipSuccess)
    {
        (void)hipGetLastError();
        throw Error(NVCV_ERROR_DEVICE, "%s failed: %s", what, hipGetErrorString(e));
    }
}

class VarShapeBatch final : public CoreObject
{
public:
    VarShapeBatch(const NVCVImageBatchVarShapeRequirements &reqs, NVCVAllocatorHandle halloc)
        : m_reqs(reqs)
        , m_alloc(ResolveAllocator(halloc, &m_hAlloc))
    {
        if (reqs.capacity < 0)
        {
            release();
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Capacity must be >= 0, not %d", reqs.capacity);
        }
        try
        {
            m_devImages   = static_cast<NVCVImageBufferStrided *>(m_alloc.allocDevice(imagesBytes(), m_reqs.alignBytes));
            m_devFormats  = static_cast<NVCVImageFormat *>(m_alloc.allocDevice(formatsBytes(), m_reqs.alignBytes));
            m_hostImages  = static_cast<NVCVImageBufferStrided *>(m_alloc.allocPinned(imagesBytes(), m_reqs.alignBytes));
            m_hostFormats = static_cast<NVCVImageFormat *>(m_alloc.allocPinned(formatsBytes(), m_reqs.alignBytes));
            m_handles     = static_cast<NVCVImageHandle *>(m_alloc.allocHost(handlesBytes(), m_reqs.alignBytes));
            CheckHip(hipEventCreateWithFlags(&m_uploaded, hipEventDisableTiming), "hipEventCreateWithFlags");
        }
        catch (...)
        {
            freeAll();
            release();
            throw;
        }
    }

    ~VarShapeBatch() override
    {
        if (m_uploaded != nullptr)
        {
            (void)hipEventSynchronize(m_uploaded);
        }
        clear();
        freeAll();
        release();
    }

    int32_t capacity() const
    {
        return m_reqs.capacity;
    }

    int32_t numImages() const
    {
        return m_num;
    }

    NVCVAllocatorHandle allocHandle() const
    {
        return m_hAlloc;
    }

    void maxSize(int32_t *w, int32_t *h)
    {
        updateCache();
        *w = m_maxW;
        *h = m_maxH;
    }

    NVCVImageFormat uniqueFormat()
    {
        updateCache();
        return m_uniqueFmt;
    }

    const NVCVImageBufferStrided *hostImages() const
    {
        return m_hostImages;
    }

    void exportData(hipStream_t stream, NVCVImageBatchData &out)
    {
        out                                       = {};
        out.numImages                             = m_num;
        out.bufferType                            = NVCV_IMAGE_BATCH_VARSHAPE_BUFFER_STRIDED_CUDA;
        NVCVImageBatchVarShapeBufferStrided &buf = out.buffer.varShapeStrided;
        buf.imageList                             = m_devImages;
        buf.formatList                            = m_devFormats;
        buf.hostFormatList                        = m_hostFormats;
        if (m_dirtyFrom < m_num)
        {
            // A stream under graph capture would record the upload and the event below into the graph: every
            // replay would then copy whatever the host mirror holds at that time, and the captured event could
            // no longer be waited on by the next push. Descriptors must be on the device before capture starts.
            hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
            if (hipStreamIsCapturing(stream, &capture) != hipSuccess)
            {
                (void)hipGetLastError(); // e.g. the legacy stream while another stream captures: not this stream's capture
                capture = hipStreamCaptureStatusNone;
            }
            if (capture != hipStreamCaptureStatusNone)
            {
                throw Error(NVCV_ERROR_INVALID_OPERATION,
                            "Image batch has %d image descriptor(s) not yet uploaded and the stream is capturing a graph: "
                            "submit the batch once (or export its data) on a stream that is not capturing first",
                            m_num - m_dirtyFrom);
            }
            // Order after any earlier upload (possibly issued on another stream), then copy the tail
            // of the arrays that changed since the last export.
            CheckHip(hipStreamWaitEvent(stream, m_uploaded, 0), "hipStreamWaitEvent");
            size_t n = (size_t)(m_num - m_dirtyFrom);
            CheckHip(hipMemcpyAsync(m_devImages + m_dirtyFrom, m_hostImages + m_dirtyFrom, n * sizeof(*m_devImages),
                                    hipMemcpyHostToDevice, stream),
                     "hipMemcpyAsync");
            CheckHip(hipMemcpyAsync(m_devFormats + m_dirtyFrom, m_hostFormats + m_dirtyFrom, n * sizeof(*m_devFormats),
                                    hipMemcpyHostToDevice, stream),
                     "hipMemcpyAsync");
            CheckHip(hipEventRecord(m_uploaded, stream), "hipEventRecord");
            m_dirtyFrom = m_num;
        }
        updateCache();
        buf.maxWidth     = m_maxW;
        buf.maxHeight    = m_maxH;
        buf.uniqueFormat = m_uniqueFmt;
    }

    void push(const NVCVImageHandle *images, int32_t n)
    {
        NotNull(images, "Images buffer");
        if (n < 0)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Number of images cannot be negative");
        }
        if ((int64_t)n + m_num > m_reqs.capacity)
        {
            throw Error(NVCV_ERROR_OVERFLOW, "Adding %d images to image batch would make its size %d exceed its capacity %d",
                        n, n + m_num, m_reqs.capacity);
        }
        waitUpload();
        int before = m_num;
        try
        {
            for (int i = 0; i < n; ++i)
            {
                pushOne(images[i]);
            }
        }
        catch (...)
        {
            rollback(before);
            throw;
        }
    }

    void pushCallback(NVCVPushImageFunc cb, void *ctx)
    {
        if (cb == nullptr)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Callback function that adds images to the image batch cannot be NULL");
        }
        waitUpload();
        int before = m_num;
        try
        {
            while (NVCVImageHandle h = cb(ctx))
            {
                if (m_num == m_reqs.capacity)
                {
                    throw Error(NVCV_ERROR_OVERFLOW,
                                "Adding one more image to image batch would make its size exceed its capacity %d",
                                m_reqs.capacity);
                }
                pushOne(h);
            }
        }
        catch (...)
        {
            rollback(before);
            throw;
        }
    }

    void pop(int32_t n)
    {
        if (n < 0)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "The number of images to remove cannot be negative");
        }
        if (n > m_num)
        {
            throw Error(NVCV_ERROR_UNDERFLOW, "Cannot remove more images, %d, than the number of images, %d, in the image batch",
                        n, m_num);
        }
        rollback(m_num - n);
    }

    void clear()
    {
        rollback(0);
        m_dirtyFrom = 0;
    }

    void getImages(int32_t beg, NVCVImageHandle *out, int32_t n) const
    {
        if (beg < 0)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Image index cannot be negative");
        }
        if (n < 0 || (int64_t)beg + n > m_num)
        {
            throw Error(NVCV_ERROR_OVERFLOW, "Cannot get images past end of image batch");
        }
        if (n > 0)
        {
            NotNull(out, "Output image handle buffer");
        }
        for (int i = 0; i < n; ++i)
        {
            out[i] = m_handles[beg + i];
            ImagePool().incRef(out[i]);
        }
    }

private:
    int64_t imagesBytes() const
    {
        return (int64_t)m_reqs.capacity * (int64_t)sizeof(NVCVImageBufferStrided);
    }

    int64_t formatsBytes() const
    {
        return (int64_t)m_reqs.capacity * (int64_t)sizeof(NVCVImageFormat);
    }

    int64_t handlesBytes() const
    {
        return (int64_t)m_reqs.capacity * (int64_t)sizeof(NVCVImageHandle);
    }

    void waitUpload()
    {
        // The pinned mirror may still be read by an in-flight upload.
        CheckHip(hipEventSynchronize(m_uploaded), "hipEventSynchronize");
    }

    void pushOne(NVCVImageHandle h)
    {
        IImage &img = Deref<IImage>(ImagePool(), h);
        if (FormatMemLayout(img.format()) != NVCV_MEM_LAYOUT_PL)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Format of image to be added must be pitch-linear");
        }
        NVCVImageData d;
        img.exportData(d);
        if (d.bufferType != NVCV_IMAGE_BUFFER_STRIDED_CUDA)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Data buffer of image to be added isn't device-accessible");
        }
        ImagePool().incRef(h);
        m_hostImages[m_num]  = d.buffer.strided;
        m_hostFormats[m_num] = d.format;
        m_handles[m_num]     = h;
        ++m_num;
        m_cacheValid = false;
    }

    // Drops images [keep, m_num).
    void rollback(int keep) noexcept
    {
        for (int i = m_num - 1; i >= keep; --i)
        {
            try
            {
                ImagePool().decRef(m_handles[i]);
            }
            catch (...)
            {
            }
            m_handles[i] = nullptr;
        }
        m_num        = keep;
        m_dirtyFrom  = std::min(m_dirtyFrom, m_num);
        m_cacheValid = false;
    }

    void updateCache()
    {
        if (m_cacheValid)
        {
            return;
        }
        m_maxW = m_maxH = 0;
        m_uniqueFmt     = NVCV_IMAGE_FORMAT_NONE;
        for (int i = 0; i < m_num; ++i)
        {
            m_maxW = std::max(m_maxW, m_hostImages[i].planes[0].width);
            m_maxH = std::max(m_maxH, m_hostImages[i].planes[0].height);
            if (i == 0)
            {
                m_uniqueFmt = m_hostFormats[0];
            }
            else if (m_uniqueFmt != m_hostFormats[i])
            {
                m_uniqueFmt = NVCV_IMAGE_FORMAT_NONE;
            }
        }
        m_cacheValid = true;
    }

    void freeAll() noexcept
    {
        m_alloc.freeDevice(m_devImages, imagesBytes(), m_reqs.alignBytes);
        m_alloc.freeDevice(m_devFormats, formatsBytes(), m_reqs.alignBytes);
        m_alloc.freePinned(m_hostImages, imagesBytes(), m_reqs.alignBytes);
        m_alloc.freePinned(m_hostFormats, formatsBytes(), m_reqs.alignBytes);
        m_alloc.freeHost(m_handles, handlesBytes(), m_reqs.alignBytes);
        if (m_uploaded != nullptr)
        {
            (void)hipEventDestroy(m_uploaded);
            m_uploaded = nullptr;
        }
    }

    void release() noexcept
    {
        if (m_hAlloc != nullptr)
        {
            try
            {
                AllocatorPool().decRef(m_hAlloc);
            }
            catch (...)
            {
            }
            m_hAlloc = nullptr;
        }
    }

    NVCVImageBatchVarShapeRequirements m_reqs;
    NVCVAllocatorHandle                m_hAlloc = nullptr;
    IAllocator                        &m_alloc;

    NVCVImageBufferStrided *m_devImages   = nullptr;
    NVCVImageFormat        *m_devFormats  = nullptr;
    NVCVImageBufferStrided *m_hostImages  = nullptr;
    NVCVImageFormat        *m_hostFormats = nullptr;
    NVCVImageHandle        *m_handles     = nullptr;
    hipEvent_t              m_uploaded    = nullptr;

    int32_t         m_num        = 0;
    int32_t         m_dirtyFrom  = 0;
    bool            m_cacheValid = false;
    int32_t         m_maxW = 0, m_maxH = 0;
    NVCVImageFormat m_uniqueFmt = NVCV_IMAGE_FORMAT_NONE;
};

VarShapeBatch &Batch(NVCVImageBatchHandle h)
{
    return Deref<VarShapeBatch>(ImageBatchPool(), h);
}

} // namespace
} // namespace nvcvamd

using namespace nvcvamd;

extern "C"
{
NVCVStatus nvcvImageBatchVarShapeCalcRequirements(int32_t capacity, NVCVImageBatchVarShapeRequirements *reqs)
{
    return Protect(
        [&]
        {
            NotNull(reqs, "Pointer to output image batch requirements");
            if (capacity < 0)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Capacity must be >= 0, not %d", capacity);
            }
            NVCVImageBatchVarShapeRequirements r = {};
            r.capacity                           = capacity;
            int64_t align = std::lcm<int64_t>(alignof(NVCVImageBufferStrided), alignof(NVCVImageHandle));
            align         = NextPow2(std::lcm<int64_t>(align, alignof(NVCVImageFormat)));
            r.alignBytes  = (int32_t)align;
            ReqAddBuffer(r.mem.cudaMem, (int64_t)capacity * sizeof(NVCVImageBufferStrided), align);
            ReqAddBuffer(r.mem.cudaMem, (int64_t)capacity * sizeof(NVCVImageFormat), align);
            ReqAddBuffer(r.mem.hostPinnedMem, (int64_t)capacity * sizeof(NVCVImageBufferStrided), align);
            ReqAddBuffer(r.mem.hostPinnedMem, (int64_t)capacity * sizeof(NVCVImageFormat), align);
            ReqAddBuffer(r.mem.hostMem, (int64_t)capacity * sizeof(NVCVImageHandle), align);
            *reqs = r;
        });
}

NVCVStatus nvcvImageBatchVarShapeConstruct(const NVCVImageBatchVarShapeRequirements *reqs, NVCVAllocatorHandle alloc,
                                           NVCVImageBatchHandle *handle)
{
    return Protect(
        [&]
        {
            NotNull(reqs, "Pointer to image batch requirements");
            NotNull(handle, "Pointer to output handle");
            *handle = static_cast<NVCVImageBatchHandle>(
                ImageBatchPool().create(std::make_unique<VarShapeBatch>(*reqs, alloc)));
        });
}

NVCVStatus nvcvImageBatchDecRef(NVCVImageBatchHandle handle, int *newRefCount)
{
    return Protect(
        [&]
        {
            int n = ImageBatchPool().decRef(handle);
            if (newRefCount)
            {
                *newRefCount = n;
            }
        });
}

NVCVStatus nvcvImageBatchIncRef(NVCVImageBatchHandle handle, int *newRefCount)
{
    return Protect(
        [&]
        {
            int n = ImageBatchPool().incRef(handle);
            if (newRefCount)
            {
                *newRefCount = n;
            }
        });
}

NVCVStatus nvcvImageBatchRefCount(NVCVImageBatchHandle handle, int *newRefCount)
{
    return Protect([&] { *NotNull(newRefCount, "Pointer to output") = ImageBatchPool().refCount(handle); });
}

NVCVStatus nvcvImageBatchSetUserPointer(NVCVImageBatchHandle handle, void *userPtr)
{
    return Protect([&] { ImageBatchPool().get(handle)->userPtr = userPtr; });
}

NVCVStatus nvcvImageBatchGetUserPointer(NVCVImageBatchHandle handle, void **outUserPtr)
{
    return Protect([&] { *NotNull(outUserPtr, "Pointer to output") = ImageBatchPool().get(handle)->userPtr; });
}

NVCVStatus nvcvImageBatchGetType(NVCVImageBatchHandle handle, NVCVTypeImageBatch *type)
{
    return Protect(
        [&]
        {
            NotNull(type, "Pointer to output");
            (void)Batch(handle);
            *type = NVCV_TYPE_IMAGEBATCH_VARSHAPE;
        });
}

NVCVStatus nvcvImageBatchGetCapacity(NVCVImageBatchHandle handle, int32_t *capacity)
{
    return Protect([&] { *NotNull(capacity, "Pointer to output capacity") = Batch(handle).capacity(); });
}

NVCVStatus nvcvImageBatchGetAllocator(NVCVImageBatchHandle handle, NVCVAllocatorHandle *alloc)
{
    return Protect(
        [&]
        {
            NotNull(alloc, "Pointer to allocator output");
            NVCVAllocatorHandle h = Batch(handle).allocHandle();
            if (h != nullptr)
            {
                AllocatorPool().incRef(h);
            }
            *alloc = h;
        });
}

NVCVStatus nvcvImageBatchGetNumImages(NVCVImageBatchHandle handle, int32_t *numImages)
{
    return Protect([&] { *NotNull(numImages, "Pointer to output") = Batch(handle).numImages(); });
}

NVCVStatus nvcvImageBatchExportData(NVCVImageBatchHandle handle, NVCVStreamHandle stream, NVCVImageBatchData *data)
{
    return Protect([&] { Batch(handle).exportData(stream, *NotNull(data, "Pointer to output data")); });
}

NVCVStatus nvcvImageBatchVarShapeGetMaxSize(NVCVImageBatchHandle handle, int32_t *maxWidth, int32_t *maxHeight)
{
    return Protect(
        [&]
        {
            if (maxWidth == nullptr && maxHeight == nullptr)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Both output width and height pointers cannot be NULL");
            }
            int32_t w, h;
            Batch(handle).maxSize(&w, &h);
            if (maxWidth)
            {
                *maxWidth = w;
            }
            if (maxHeight)
            {
                *maxHeight = h;
            }
        });
}

NVCVStatus nvcvImageBatchVarShapeGetUniqueFormat(NVCVImageBatchHandle handle, NVCVImageFormat *format)
{
    return Protect([&] { *NotNull(format, "Pointer to output format") = Batch(handle).uniqueFormat(); });
}

NVCVStatus nvcvImageBatchVarShapePushImages(NVCVImageBatchHandle handle, const NVCVImageHandle *images, int32_t numImages)
{
    return Protect([&] { Batch(handle).push(images, numImages); });
}

NVCVStatus nvcvImageBatchVarShapePushImagesCallback(NVCVImageBatchHandle handle, NVCVPushImageFunc cbPushImage,
                                                    void *ctxCallback)
{
    return Protect([&] { Batch(handle).pushCallback(cbPushImage, ctxCallback); });
}

NVCVStatus nvcvImageBatchVarShapePopImages(NVCVImageBatchHandle handle, int32_t numImages)
{
    return Protect([&] { Batch(handle).pop(numImages); });
}

NVCVStatus nvcvImageBatchVarShapeClear(NVCVImageBatchHandle handle)
{
    return Protect([&] { Batch(handle).clear(); });
}

NVCVStatus nvcvImageBatchVarShapeGetImages(NVCVImageBatchHandle handle, int32_t begIndex, NVCVImageHandle *outImages,
                                           int32_t numImages)
{
    return Protect([&] { Batch(handle).getImages(begIndex, outImages, numImages); });
}

NVCVStatus nvcvxImageBatchVarShapeGetHostImageList(NVCVImageBatchHandle handle, const NVCVImageBufferStrided **outList,
                                                   int32_t *outNumImages)
{
    return Protect(
        [&]
        {
            VarShapeBatch &b                                  = Batch(handle);
            *NotNull(outList, "Pointer to output list")       = b.hostImages();
            *NotNull(outNumImages, "Pointer to output count") = b.numImages();
        });
}
}
