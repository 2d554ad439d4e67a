// Image objects: owning images (all planes in one device allocation) and wrapped images.
// Behaviour follows src/nvcv/src/priv/Image.cpp:36-262 of the reference; row/base alignment
// defaults are this library's constants (128 B / 512 B) so requirement queries need no device.
#include "Priv.hpp"

#include <algorithm>
#include <numeric>

namespace nvcvamd {

namespace {

NVCVImageRequirements CalcImageRequirements(int32_t w, int32_t h, uint64_t fmt, int32_t userBaseAlign,
                                            int32_t userRowAlign)
{
    if (w < 0 || h < 0)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Image size must be >= 0, not %dx%d", w, h);
    }
    int planes = FormatNumPlanes(fmt);
    if (planes < 1)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Image format has no planes");
    }
    NVCVImageRequirements reqs = {};
    reqs.width                 = w;
    reqs.height                = h;
    reqs.format                = fmt;

    int64_t rowAlign;
    if (userRowAlign == 0)
    {
        rowAlign = kDefaultRowAlign;
    }
    else
    {
        if (!IsPow2(userRowAlign))
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Invalid pitch alignment of %d, it must be a power-of-two",
                        userRowAlign);
        }
        rowAlign = userRowAlign;
    }
    for (int p = 0; p < planes; ++p)
    {
        rowAlign = std::lcm<int64_t>(rowAlign, DataTypeAlignment(FormatPlaneDataType(fmt, p)));
    }
    rowAlign = NextPow2(rowAlign);

    int64_t baseAlign;
    if (userBaseAlign == 0)
    {
        baseAlign = kDefaultBaseAlign;
    }
    else
    {
        if (!IsPow2(userBaseAlign))
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Invalid buffer address alignment of %d, it must be a power-of-two",
                        userBaseAlign);
        }
        baseAlign = userBaseAlign;
    }
    baseAlign = std::lcm<int64_t>(baseAlign, rowAlign);
    if (baseAlign >= NVCV_MAX_MEM_REQUIREMENTS_BLOCK_SIZE)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Alignment requirement of %ld is too large", (long)baseAlign);
    }
    reqs.alignBytes = (int32_t)baseAlign;

    for (int p = 0; p < planes; ++p)
    {
        int32_t pw, ph;
        FormatPlaneSize(fmt, p, w, h, &pw, &ph);
        int64_t pitch = AlignUp((int64_t)pw * FormatPlanePixelStrideBytes(fmt, p), rowAlign);
        if (pitch > INT32_MAX)
        {
            throw Error(NVCV_ERROR_OVERFLOW, "Row pitch of plane %d does not fit in 32 bits", p);
        }
        reqs.planeRowStride[p] = (int32_t)pitch;
        ReqAddBuffer(reqs.mem.cudaMem, pitch * ph, baseAlign);
    }
    return reqs;
}

class OwningImage final : public IImage
{
public:
    OwningImage(const NVCVImageRequirements &reqs, NVCVAllocatorHandle halloc)
        : m_reqs(reqs)
        , m_alloc(ResolveAllocator(halloc, &m_hAlloc))
    {
        try
        {
            if (FormatMemLayout(m_reqs.format) != NVCV_MEM_LAYOUT_PL)
            {
                throw Error(NVCV_ERROR_NOT_IMPLEMENTED, "Image with block-linear format is not supported");
            }
            m_bytes = ReqTotalBytes(m_reqs.mem.cudaMem);
            m_mem   = m_alloc.allocDevice(m_bytes, m_reqs.alignBytes);
        }
        catch (...)
        {
            release();
            throw;
        }
    }

    ~OwningImage() override
    {
        m_alloc.freeDevice(m_mem, m_bytes, m_reqs.alignBytes);
        release();
    }

    NVCVTypeImage type() const override
    {
        return NVCV_TYPE_IMAGE;
    }

    void size(int32_t *w, int32_t *h) const override
    {
        *w = m_reqs.width;
        *h = m_reqs.height;
    }

    NVCVImageFormat format() const override
    {
        return m_reqs.format;
    }

    void exportData(NVCVImageData &out) const override
    {
        out                         = {};
        out.format                  = m_reqs.format;
        out.bufferType              = NVCV_IMAGE_BUFFER_STRIDED_CUDA;
        NVCVImageBufferStrided &buf = out.buffer.strided;
        buf.numPlanes               = FormatNumPlanes(m_reqs.format);
        // Planes follow each other without gaps (reference: src/nvcv/src/priv/Image.cpp:174-187): plane p + 1
        // starts row pitch x height after plane p, so a planar image is also a dense CHW block. The requirements
        // sum one aligned block run per plane, which is never less.
        int64_t offset = 0;
        for (int p = 0; p < buf.numPlanes; ++p)
        {
            NVCVImagePlaneStrided &pl = buf.planes[p];
            FormatPlaneSize(m_reqs.format, p, m_reqs.width, m_reqs.height, &pl.width, &pl.height);
            pl.rowStride = m_reqs.planeRowStride[p];
            pl.basePtr   = static_cast<NVCVByte *>(m_mem) + offset;
            offset += (int64_t)pl.rowStride * pl.height;
        }
    }

    NVCVAllocatorHandle allocHandle() const override
    {
        return m_hAlloc;
    }

private:
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

    NVCVImageRequirements m_reqs;
    NVCVAllocatorHandle   m_hAlloc = nullptr;
    IAllocator           &m_alloc;
    void                 *m_mem   = nullptr;
    int64_t               m_bytes = 0;
};

class WrappedImage final : public IImage
{
public:
    WrappedImage(const NVCVImageData &d, NVCVImageDataCleanupFunc cleanup, void *ctx)
        : m_data(d)
        , m_cleanup(cleanup)
        , m_ctx(ctx)
    {
        switch (d.bufferType)
        {
        case NVCV_IMAGE_BUFFER_STRIDED_CUDA:
            break;
        case NVCV_IMAGE_BUFFER_STRIDED_HOST:
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Wrapping of host memory into an image isn't supported");
        case NVCV_IMAGE_BUFFER_CUDA_ARRAY:
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Wrapping of texture arrays into an image isn't supported");
        default:
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Invalid wrapping of buffer type NONE");
        }
        if (FormatMemLayout(d.format) != NVCV_MEM_LAYOUT_PL)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Pitch-linear buffer not consistent with image format %s",
                        nvcvImageFormatGetName(d.format));
        }
        const NVCVImageBufferStrided &buf = d.buffer.strided;
        if (buf.numPlanes < 1 || buf.numPlanes > NVCV_MAX_PLANE_COUNT)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Number of planes must be in [1,%d], not %d", NVCV_MAX_PLANE_COUNT,
                        buf.numPlanes);
        }
        for (int p = 0; p < buf.numPlanes; ++p)
        {
            const NVCVImagePlaneStrided &pl = buf.planes[p];
            if (pl.width < 1 || pl.height < 1)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Plane #%d must have dimensions >= 1x1, not %dx%d", p, pl.width,
                            pl.height);
            }
            if (pl.basePtr == nullptr)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Plane #%d's base pointer must not be NULL", p);
            }
        }
    }

    ~WrappedImage() override
    {
        if (m_cleanup != nullptr)
        {
            m_cleanup(m_ctx, &m_data);
        }
    }

    NVCVTypeImage type() const override
    {
        return NVCV_TYPE_IMAGE_WRAPDATA;
    }

    void size(int32_t *w, int32_t *h) const override
    {
        *w = m_data.buffer.strided.planes[0].width;
        *h = m_data.buffer.strided.planes[0].height;
    }

    NVCVImageFormat format() const override
    {
        return m_data.format;
    }

    void exportData(NVCVImageData &out) const override
    {
        out = m_data;
    }

    NVCVAllocatorHandle allocHandle() const override
    {
        return nullptr;
    }

private:
    NVCVImageData            m_data;
    NVCVImageDataCleanupFunc m_cleanup;
    void                    *m_ctx;
};

} // namespace
} // namespace nvcvamd

using namespace nvcvamd;

extern "C"
{
NVCVStatus nvcvImageCalcRequirements(int32_t width, int32_t height, NVCVImageFormat format, int32_t baseAddrAlignment,
                                     int32_t rowAddrAlignment, NVCVImageRequirements *reqs)
{
    return Protect(
        [&]
        {
            NotNull(reqs, "Pointer to output image requirements");
            *reqs = CalcImageRequirements(width, height, format, baseAddrAlignment, rowAddrAlignment);
        });
}

NVCVStatus nvcvImageConstruct(const NVCVImageRequirements *reqs, NVCVAllocatorHandle alloc, NVCVImageHandle *handle)
{
    return Protect(
        [&]
        {
            NotNull(reqs, "Pointer to image requirements");
            NotNull(handle, "Pointer to output handle");
            *handle = static_cast<NVCVImageHandle>(ImagePool().create(std::make_unique<OwningImage>(*reqs, alloc)));
        });
}

NVCVStatus nvcvImageWrapDataConstruct(const NVCVImageData *data, NVCVImageDataCleanupFunc cleanup, void *ctxCleanup,
                                      NVCVImageHandle *handle)
{
    return Protect(
        [&]
        {
            NotNull(data, "Pointer to image data");
            NotNull(handle, "Pointer to output handle");
            *handle = static_cast<NVCVImageHandle>(
                ImagePool().create(std::make_unique<WrappedImage>(*data, cleanup, ctxCleanup)));
        });
}

NVCVStatus nvcvImageDecRef(NVCVImageHandle handle, int *newRefCount)
{
    return Protect(
        [&]
        {
            int n = ImagePool().decRef(handle);
            if (newRefCount)
            {
                *newRefCount = n;
            }
        });
}

NVCVStatus nvcvImageIncRef(NVCVImageHandle handle, int *newRefCount)
{
    return Protect(
        [&]
        {
            int n = ImagePool().incRef(handle);
            if (newRefCount)
            {
                *newRefCount = n;
            }
        });
}

NVCVStatus nvcvImageRefCount(NVCVImageHandle handle, int *newRefCount)
{
    return Protect([&] { *NotNull(newRefCount, "Pointer to output") = ImagePool().refCount(handle); });
}

NVCVStatus nvcvImageSetUserPointer(NVCVImageHandle handle, void *userPtr)
{
    return Protect([&] { ImagePool().get(handle)->userPtr = userPtr; });
}

NVCVStatus nvcvImageGetUserPointer(NVCVImageHandle handle, void **outUserPtr)
{
    return Protect([&] { *NotNull(outUserPtr, "Pointer to output") = ImagePool().get(handle)->userPtr; });
}

NVCVStatus nvcvImageGetType(NVCVImageHandle handle, NVCVTypeImage *type)
{
    return Protect([&] { *NotNull(type, "Pointer to output") = Deref<IImage>(ImagePool(), handle).type(); });
}

NVCVStatus nvcvImageGetSize(NVCVImageHandle handle, int32_t *width, int32_t *height)
{
    return Protect(
        [&]
        {
            NotNull(width, "Pointer to width output");
            NotNull(height, "Pointer to height output");
            Deref<IImage>(ImagePool(), handle).size(width, height);
        });
}

NVCVStatus nvcvImageGetFormat(NVCVImageHandle handle, NVCVImageFormat *fmt)
{
    return Protect([&] { *NotNull(fmt, "Pointer to format output") = Deref<IImage>(ImagePool(), handle).format(); });
}

NVCVStatus nvcvImageGetAllocator(NVCVImageHandle handle, NVCVAllocatorHandle *alloc)
{
    return Protect(
        [&]
        {
            NotNull(alloc, "Pointer to allocator output");
            NVCVAllocatorHandle h = Deref<IImage>(ImagePool(), handle).allocHandle();
            if (h != nullptr)
            {
                AllocatorPool().incRef(h);
            }
            *alloc = h;
        });
}

NVCVStatus nvcvImageExportData(NVCVImageHandle handle, NVCVImageData *data)
{
    return Protect([&] { Deref<IImage>(ImagePool(), handle).exportData(*NotNull(data, "Pointer to image data output")); });
}
}
