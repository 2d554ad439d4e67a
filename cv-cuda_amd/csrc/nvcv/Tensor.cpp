// Tensor objects: stride computation, owning and wrapping tensors, reshape views.
// Stride rule and validation follow the reference (src/nvcv/src/priv/Tensor.cpp:41-190,
// TensorWrapDataStrided.cpp:35-105, TensorData.cpp:30-48, 286-350); the alignment constants are this
// library's own (128-byte rows, 512-byte base) instead of CUDA texture attributes, so requirement
// queries need no device.
#include "Priv.hpp"

#include <algorithm>
#include <cstring>
#include <numeric>

namespace nvcvamd {

namespace {

NVCVTensorRequirements CalcRequirements(int32_t rank, const int64_t *shape, NVCVDataType dtype,
                                        NVCVTensorLayout layout, int32_t userBaseAlign, int32_t userRowAlign)
{
    NVCVTensorRequirements reqs = {};
    reqs.layout                 = layout;
    reqs.dtype                  = dtype;

    if (layout.rank > 0 && rank != layout.rank)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Number of shape dimensions %d must be equal to layout dimensions %d",
                    rank, layout.rank);
    }
    if (rank <= 0 || rank > NVCV_TENSOR_MAX_RANK)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Number of dimensions must be in [1,%d], not %d", NVCV_TENSOR_MAX_RANK,
                    rank);
    }
    NotNull(shape, "Pointer to shape");
    int elemBytes = DataTypeStrideBytes(dtype);
    if (elemBytes <= 0)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Data type has no storage size");
    }
    for (int i = 0; i < rank; ++i)
    {
        if (shape[i] < 0)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Shape #%d must be >= 0, not %ld", i, (long)shape[i]);
        }
        reqs.shape[i] = shape[i];
    }
    reqs.rank = rank;

    int64_t rowAlign;
    if (userRowAlign == 0)
    {
        rowAlign = std::lcm<int64_t>(kDefaultRowAlign, NextPow2(elemBytes));
    }
    else
    {
        if (!IsPow2(userRowAlign))
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Invalid pitch alignment of %d, it must be a power-of-two",
                        userRowAlign);
        }
        rowAlign = std::lcm<int64_t>(userRowAlign, DataTypeAlignment(dtype));
    }

    int64_t baseAlign;
    if (userBaseAlign == 0)
    {
        baseAlign = NextPow2(std::lcm<int64_t>(kDefaultBaseAlign, rowAlign));
    }
    else
    {
        if (!IsPow2(userBaseAlign))
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Invalid base address alignment of %d, it must be a power-of-two",
                        userBaseAlign);
        }
        baseAlign = std::lcm<int64_t>(rowAlign, userBaseAlign);
    }
    if (baseAlign >= NVCV_MAX_MEM_REQUIREMENTS_BLOCK_SIZE)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Alignment requirement of %ld is too large", (long)baseAlign);
    }
    reqs.alignBytes = (int32_t)baseAlign;

    // Dimensions [firstPacked, rank) are contiguous; the one just outside is padded to rowAlign.
    NVCVTensorLayout last2       = LayoutLast(layout, 2);
    int              firstPacked = (last2.rank == 2 && last2.data[0] == 'W' && last2.data[1] == 'C') ? std::max(0, rank - 2)
                                                                                                    : rank - 1;
    reqs.strides[rank - 1] = elemBytes;
    for (int d = rank - 2; d >= 0; --d)
    {
        int64_t packed  = reqs.shape[d + 1] * reqs.strides[d + 1];
        reqs.strides[d] = (d == firstPacked - 1) ? AlignUp(packed, rowAlign) : packed;
    }
    ReqAddBuffer(reqs.mem.cudaMem, reqs.strides[0] * reqs.shape[0], reqs.alignBytes);
    return reqs;
}

NVCVTensorLayout LayoutForImages(uint64_t fmt, int numImages)
{
    int planes = FormatNumPlanes(fmt);
    (void)numImages; // a single image still gets a batch dimension
    if (planes == 1)
    {
        return NVCV_TENSOR_NHWC;
    }
    if (planes == FormatNumChannels(fmt))
    {
        return NVCV_TENSOR_NCHW;
    }
    throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Image format cannot be semi-planar, but it is: %s",
                nvcvImageFormatGetName(fmt));
}

// Element type of a tensor holding images of format `fmt`: the first component of plane 0 on its own, when a
// packing of just that many bits exists (reference: src/nvcv/src/priv/Tensor.cpp:79-91).
NVCVDataType ChannelDataTypeOf(uint64_t fmt)
{
    NVCVPackingParams params;
    NVCVPacking       one;
    if (nvcvPackingGetParams(FormatPlanePacking(fmt, 0), &params) != NVCV_SUCCESS)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Image format can't be represented in a tensor: %s",
                    nvcvImageFormatGetName(fmt));
    }
    params.swizzle = NVCV_SWIZZLE_X000;
    std::fill(params.bits + 1, params.bits + 4, 0);
    if (nvcvMakePacking(&one, &params) != NVCV_SUCCESS)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Image format can't be represented in a tensor: %s",
                    nvcvImageFormatGetName(fmt));
    }
    return NVCV_DETAIL_MAKE_DATA_TYPE(FormatDataKind(fmt), (uint64_t)one);
}

NVCVTensorRequirements CalcRequirementsForImages(int32_t numImages, int32_t w, int32_t h, uint64_t fmt,
                                                 int32_t baseAlign, int32_t rowAlign)
{
    if (FormatMemLayout(fmt) != NVCV_MEM_LAYOUT_PL)
    {
        throw Error(NVCV_ERROR_NOT_IMPLEMENTED, "Tensor image batch of block-linear format images is not supported");
    }
    if (FormatCSS(fmt) != NVCV_CSS_444)
    {
        throw Error(NVCV_ERROR_NOT_IMPLEMENTED, "Batch image format must not have subsampled planes, but it is: %s",
                    nvcvImageFormatGetName(fmt));
    }
    int planes = FormatNumPlanes(fmt);
    if (planes != 1 && planes != FormatNumChannels(fmt))
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Image format cannot be semi-planar, but it is: %s",
                    nvcvImageFormatGetName(fmt));
    }
    for (int p = 1; p < planes; ++p)
    {
        if (FormatPlanePacking(fmt, p) != FormatPlanePacking(fmt, 0))
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Format's planes must all have the same packing: %s",
                        nvcvImageFormatGetName(fmt));
        }
    }
    NVCVTensorLayout layout       = LayoutForImages(fmt, numImages);
    int64_t          shapeNCHW[4] = {numImages, FormatNumChannels(fmt), h, w};
    int64_t          shape[NVCV_TENSOR_MAX_RANK];
    PermuteShape(NVCV_TENSOR_NCHW, shapeNCHW, layout, shape);
    return CalcRequirements(layout.rank, shape, ChannelDataTypeOf(fmt), layout, baseAlign, rowAlign);
}

class OwningTensor final : public ITensor
{
public:
    OwningTensor(const NVCVTensorRequirements &reqs, NVCVAllocatorHandle halloc)
        : m_reqs(reqs)
        , m_alloc(ResolveAllocator(halloc, &m_hAlloc))
    {
        try
        {
            m_bytes = ReqTotalBytes(m_reqs.mem.cudaMem);
            m_mem   = m_alloc.allocDevice(m_bytes, m_reqs.alignBytes);
        }
        catch (...)
        {
            releaseAllocator();
            throw;
        }
    }

    ~OwningTensor() override
    {
        m_alloc.freeDevice(m_mem, m_bytes, m_reqs.alignBytes);
        releaseAllocator();
    }

    void exportData(NVCVTensorData &out) const override
    {
        out            = {};
        out.bufferType = NVCV_TENSOR_BUFFER_STRIDED_CUDA;
        out.dtype      = m_reqs.dtype;
        out.layout     = m_reqs.layout;
        out.rank       = m_reqs.rank;
        std::copy_n(m_reqs.shape, NVCV_TENSOR_MAX_RANK, out.shape);
        std::copy_n(m_reqs.strides, NVCV_TENSOR_MAX_RANK, out.buffer.strided.strides);
        out.buffer.strided.basePtr = static_cast<NVCVByte *>(m_mem);
    }

    NVCVAllocatorHandle allocHandle() const override
    {
        return m_hAlloc;
    }

private:
    void releaseAllocator() noexcept
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

    NVCVTensorRequirements m_reqs;
    NVCVAllocatorHandle    m_hAlloc = nullptr;
    IAllocator            &m_alloc;
    void                  *m_mem   = nullptr;
    int64_t                m_bytes = 0;
};

class WrappedTensor final : public ITensor
{
public:
    WrappedTensor(const NVCVTensorData &d, NVCVTensorDataCleanupFunc cleanup, void *ctx)
        : m_data(d)
        , m_cleanup(cleanup)
        , m_ctx(ctx)
    {
        ValidateWrappedTensor(d);
    }

    ~WrappedTensor() override
    {
        if (m_cleanup != nullptr)
        {
            m_cleanup(m_ctx, &m_data);
        }
    }

    void exportData(NVCVTensorData &out) const override
    {
        out = m_data;
    }

    NVCVAllocatorHandle allocHandle() const override
    {
        return nullptr;
    }

private:
    NVCVTensorData            m_data;
    NVCVTensorDataCleanupFunc m_cleanup;
    void                     *m_ctx;
};

// Computes strides of `newShape` viewing memory described by (shape, strides), numpy-style: runs of
// input dimensions that are contiguous with each other are merged, and every merged run must be
// covered exactly by consecutive output dimensions. Unit dimensions of the input take no part in the
// merge whatever their stride says (an element of such a dimension is never stepped over), which is more
// lenient than the reference: its merge (src/nvcv/src/priv/TensorData.cpp:196-246) lets a unit dimension
// with a stride that does not continue its neighbours split a run, and then refuses the reshape.
bool ViewStrides(int rank, const int64_t *shape, const int64_t *strides, int newRank, const int64_t *newShape,
                 int64_t *newStrides)
{
    // merge
    int64_t gshape[NVCV_TENSOR_MAX_RANK], gstride[NVCV_TENSOR_MAX_RANK];
    int     ng = 0;
    for (int d = 0; d < rank; ++d)
    {
        if (shape[d] == 1)
        {
            continue;
        }
        if (ng > 0 && gstride[ng - 1] == shape[d] * strides[d])
        {
            gshape[ng - 1] *= shape[d];
            gstride[ng - 1] = strides[d];
        }
        else
        {
            gshape[ng]  = shape[d];
            gstride[ng] = strides[d];
            ++ng;
        }
    }
    if (ng == 0) // nothing but unit dimensions
    {
        gshape[0]  = 1;
        gstride[0] = strides[rank - 1];
        ng         = 1;
    }
    // Every group is split into the next output dimensions whose product is its extent; unit dimensions go with
    // the group at hand, also when its extent is already reached, and a dimension's stride is the group's stride
    // times the extents after it inside the group (reference: src/nvcv/src/priv/TensorData.cpp:248-276).
    int d = 0;
    for (int g = 0; g < ng && d < newRank; ++g)
    {
        int64_t   vol   = 1;
        const int first = d;
        while (d < newRank && vol * newShape[d] <= gshape[g])
        {
            vol *= newShape[d];
            ++d;
        }
        if (vol != gshape[g])
        {
            return false;
        }
        int64_t st = gstride[g];
        for (int k = d - 1; k >= first; --k)
        {
            newStrides[k] = st;
            st *= newShape[k];
        }
        if (g == ng - 1 && d != newRank)
        {
            return false; // equal volumes make this unreachable; kept as a guard
        }
    }
    return d == newRank;
}

} // namespace

void ValidateWrappedTensor(const NVCVTensorData &d)
{
    if (d.bufferType != NVCV_TENSOR_BUFFER_STRIDED_CUDA)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Tensor buffer type not supported, must be a device-accessible strided buffer");
    }
    const NVCVTensorBufferStrided &buf = d.buffer.strided;
    if (buf.basePtr == nullptr)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Memory buffer must not be NULL");
    }
    int rank = d.rank;
    if (rank <= 0 || rank > NVCV_TENSOR_MAX_RANK)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Number of dimensions must be in [1,%d], not %d", NVCV_TENSOR_MAX_RANK,
                    rank);
    }
    if (d.layout.rank > 0 && d.layout.rank != rank)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Layout has %d dimensions but the shape has %d", d.layout.rank, rank);
    }
    for (int i = 0; i < rank; ++i)
    {
        if (d.shape[i] < 1)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Shape #%d must be >= 1, not %ld", i, (long)d.shape[i]);
        }
    }
    int     elemBytes   = DataTypeStrideBytes(d.dtype);
    bool    channelLast = d.layout.rank == 0 || d.layout.data[d.layout.rank - 1] == 'C';
    int     firstPacked = channelLast ? std::max(0, rank - 2) : rank - 1;
    int64_t prevStride  = buf.strides[rank - 1];
    int64_t prevSize    = d.shape[rank - 1];
    int     dim         = rank - 1;
    for (; dim >= firstPacked; --dim)
    {
        if (d.shape[dim] <= 1)
        {
            continue;
        }
        int64_t want = dim == rank - 1 ? elemBytes : prevStride * prevSize;
        if (buf.strides[dim] != want)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Pitch of dimension %d must be == %ld (packed), but it is %ld", dim,
                        (long)want, (long)buf.strides[dim]);
        }
        prevStride = buf.strides[dim];
        prevSize   = d.shape[dim];
    }
    for (; dim >= 0; --dim)
    {
        if (d.shape[dim] <= 1)
        {
            continue;
        }
        int64_t minPitch = prevStride * prevSize;
        if (buf.strides[dim] < minPitch)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Pitch of dimension %d must be >= %ld, but it is %ld", dim,
                        (long)minPitch, (long)buf.strides[dim]);
        }
        prevStride = buf.strides[dim];
        prevSize   = d.shape[dim];
    }
}

} // namespace nvcvamd

using namespace nvcvamd;

namespace {
NVCVTensorHandle MakeWrapped(const NVCVTensorData &d, NVCVTensorDataCleanupFunc cleanup, void *ctx)
{
    return static_cast<NVCVTensorHandle>(TensorPool().create(std::make_unique<WrappedTensor>(d, cleanup, ctx)));
}
} // namespace

extern "C"
{
NVCVStatus nvcvTensorCalcRequirements(int32_t rank, const int64_t *shape, NVCVDataType dtype, NVCVTensorLayout layout,
                                      int32_t baseAddrAlignment, int32_t rowAddrAlignment, NVCVTensorRequirements *reqs)
{
    return Protect(
        [&]
        {
            NotNull(reqs, "Pointer to output requirements");
            *reqs = CalcRequirements(rank, shape, dtype, layout, baseAddrAlignment, rowAddrAlignment);
        });
}

NVCVStatus nvcvTensorCalcRequirementsForImages(int32_t numImages, int32_t width, int32_t height, NVCVImageFormat format,
                                               int32_t baseAddrAlignment, int32_t rowAddrAlignment,
                                               NVCVTensorRequirements *reqs)
{
    return Protect(
        [&]
        {
            NotNull(reqs, "Pointer to output requirements");
            *reqs = CalcRequirementsForImages(numImages, width, height, format, baseAddrAlignment, rowAddrAlignment);
        });
}

NVCVStatus nvcvTensorConstruct(const NVCVTensorRequirements *reqs, NVCVAllocatorHandle alloc, NVCVTensorHandle *handle)
{
    return Protect(
        [&]
        {
            NotNull(reqs, "Pointer to requirements");
            NotNull(handle, "Pointer to output handle");
            *handle = static_cast<NVCVTensorHandle>(TensorPool().create(std::make_unique<OwningTensor>(*reqs, alloc)));
        });
}

NVCVStatus nvcvTensorWrapDataConstruct(const NVCVTensorData *data, NVCVTensorDataCleanupFunc cleanup, void *ctxCleanup,
                                       NVCVTensorHandle *handle)
{
    return Protect(
        [&]
        {
            NotNull(data, "Pointer to tensor data");
            NotNull(handle, "Pointer to output handle");
            *handle = MakeWrapped(*data, cleanup, ctxCleanup);
        });
}

NVCVStatus nvcvTensorWrapImageConstruct(NVCVImageHandle himg, NVCVTensorHandle *handle)
{
    return Protect(
        [&]
        {
            NotNull(handle, "Pointer to output handle");
            IImage       &img = Deref<IImage>(ImagePool(), himg);
            NVCVImageData id;
            img.exportData(id);
            if (id.bufferType != NVCV_IMAGE_BUFFER_STRIDED_CUDA)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Only device-accessible pitch-linear images can be wrapped");
            }
            // The checks and the layout rule of the reference (src/nvcv/src/priv/TensorData.cpp:50-192).
            uint64_t fmt    = id.format;
            int      planes = id.buffer.strided.numPlanes;
            if (FormatMemLayout(fmt) != NVCV_MEM_LAYOUT_PL)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Image format's memory layout must be pitch-linear");
            }
            if (FormatCSS(fmt) != NVCV_CSS_444)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Images with subsampled planes cannot be viewed as a tensor");
            }
            const NVCVImagePlaneStrided &p0 = id.buffer.strided.planes[0];
            for (int p = 1; p < planes; ++p)
            {
                const NVCVImagePlaneStrided &pl = id.buffer.strided.planes[p];
                if (FormatPlaneDataType(fmt, p) != FormatPlaneDataType(fmt, 0))
                {
                    throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Data type of all image planes must be the same");
                }
                if (pl.rowStride != p0.rowStride || pl.width != p0.width || pl.height != p0.height)
                {
                    throw Error(NVCV_ERROR_INVALID_ARGUMENT, "All image planes must share size and row pitch");
                }
                if (pl.basePtr <= p0.basePtr)
                {
                    throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Consecutive image planes must have increasing memory addresses");
                }
                if (pl.basePtr - id.buffer.strided.planes[p - 1].basePtr
                    != id.buffer.strided.planes[1].basePtr - p0.basePtr)
                {
                    throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Image planes must be equally spaced in memory");
                }
            }
            NVCVTensorData td = {};
            td.bufferType     = NVCV_TENSOR_BUFFER_STRIDED_CUDA;
            td.rank           = 4;
            td.buffer.strided.basePtr = p0.basePtr;
            const int   ch         = FormatNumChannels(fmt);
            const int   pixelBytes = FormatPlanePixelStrideBytes(fmt, 0);
            PackingInfo pi         = DecodePacking(FormatPlanePacking(fmt, 0));
            bool        sameBits   = true;
            for (int c = 1; c < ch && c < 4; ++c)
            {
                sameBits = sameBits && pi.bits[c] == pi.bits[0];
            }
            if (planes == 1 && ch >= 2 && sameBits)
            {
                // equal channels of one interleaved plane become a dimension of their own
                td.layout = NVCV_TENSOR_NHWC;
                if (nvcvDataTypeGetChannelType(FormatPlaneDataType(fmt, 0), 0, &td.dtype) != NVCV_SUCCESS)
                {
                    throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Image format can't be represented in a tensor: %s",
                                nvcvImageFormatGetName(fmt));
                }
                int64_t shape[4]   = {1, p0.height, p0.width, ch};
                int64_t strides[4] = {(int64_t)p0.rowStride * p0.height, p0.rowStride, pixelBytes, pixelBytes / ch};
                std::copy_n(shape, 4, td.shape);
                std::copy_n(strides, 4, td.buffer.strided.strides);
            }
            else
            {
                // one element per pixel of a plane (a one-channel plane, or a pixel whose fields differ in width).
                // The plane pitch is the planes' real distance; for planes placed back to back, as image objects
                // of this library place them, that is row pitch x height.
                td.layout           = NVCV_TENSOR_NCHW;
                td.dtype            = FormatPlaneDataType(fmt, 0);
                int64_t planeStride = planes > 1 ? id.buffer.strided.planes[1].basePtr - p0.basePtr
                                                 : (int64_t)p0.rowStride * p0.height;
                int64_t shape[4]    = {1, planes, p0.height, p0.width};
                int64_t strides[4]  = {planeStride * planes, planeStride, p0.rowStride, pixelBytes};
                std::copy_n(shape, 4, td.shape);
                std::copy_n(strides, 4, td.buffer.strided.strides);
            }
            ImagePool().incRef(himg);
            try
            {
                *handle = MakeWrapped(
                    td,
                    [](void *ctx, const NVCVTensorData *)
                    {
                        try
                        {
                            ImagePool().decRef(ctx);
                        }
                        catch (...)
                        {
                        }
                    },
                    himg);
            }
            catch (...)
            {
                ImagePool().decRef(himg);
                throw;
            }
        });
}

NVCVStatus nvcvTensorDecRef(NVCVTensorHandle handle, int *newRefCount)
{
    return Protect(
        [&]
        {
            int n = TensorPool().decRef(handle);
            if (newRefCount)
            {
                *newRefCount = n;
            }
        });
}

NVCVStatus nvcvTensorIncRef(NVCVTensorHandle handle, int *newRefCount)
{
    return Protect(
        [&]
        {
            int n = TensorPool().incRef(handle);
            if (newRefCount)
            {
                *newRefCount = n;
            }
        });
}

NVCVStatus nvcvTensorRefCount(NVCVTensorHandle handle, int *newRefCount)
{
    return Protect([&] { *NotNull(newRefCount, "Pointer to output") = TensorPool().refCount(handle); });
}

NVCVStatus nvcvTensorSetUserPointer(NVCVTensorHandle handle, void *userPtr)
{
    return Protect([&] { TensorPool().get(handle)->userPtr = userPtr; });
}

NVCVStatus nvcvTensorGetUserPointer(NVCVTensorHandle handle, void **outUserPtr)
{
    return Protect([&] { *NotNull(outUserPtr, "Pointer to output") = TensorPool().get(handle)->userPtr; });
}

NVCVStatus nvcvTensorGetDataType(NVCVTensorHandle handle, NVCVDataType *type)
{
    return Protect(
        [&]
        {
            NotNull(type, "Pointer to data type output");
            NVCVTensorData d;
            Deref<ITensor>(TensorPool(), handle).exportData(d);
            *type = d.dtype;
        });
}

NVCVStatus nvcvTensorGetLayout(NVCVTensorHandle handle, NVCVTensorLayout *layout)
{
    return Protect(
        [&]
        {
            NotNull(layout, "Pointer to layout output");
            NVCVTensorData d;
            Deref<ITensor>(TensorPool(), handle).exportData(d);
            *layout = d.layout;
        });
}

NVCVStatus nvcvTensorGetAllocator(NVCVTensorHandle handle, NVCVAllocatorHandle *alloc)
{
    return Protect(
        [&]
        {
            NotNull(alloc, "Pointer to allocator output");
            NVCVAllocatorHandle h = Deref<ITensor>(TensorPool(), handle).allocHandle();
            if (h != nullptr)
            {
                AllocatorPool().incRef(h);
            }
            *alloc = h;
        });
}

NVCVStatus nvcvTensorExportData(NVCVTensorHandle handle, NVCVTensorData *data)
{
    return Protect([&] { Deref<ITensor>(TensorPool(), handle).exportData(*NotNull(data, "Pointer to tensor data output")); });
}

NVCVStatus nvcvTensorGetShape(NVCVTensorHandle handle, int32_t *rank, int64_t *shape)
{
    return Protect(
        [&]
        {
            ITensor &t = Deref<ITensor>(TensorPool(), handle);
            NotNull(rank, "Input pointer to rank");
            NVCVTensorData d;
            t.exportData(d);
            if (shape != nullptr)
            {
                int n = std::min(*rank, d.rank);
                if (n > 0)
                {
                    std::fill_n(shape, *rank - n, int64_t(1));
                    std::copy_n(d.shape + d.rank - n, n, shape + *rank - n);
                }
            }
            *rank = d.rank;
        });
}

NVCVStatus nvcvTensorReshape(NVCVTensorHandle handle, int32_t rank, const int64_t *shape, NVCVTensorLayout layout,
                             NVCVTensorHandle *out_handle)
{
    return Protect(
        [&]
        {
            NotNull(out_handle, "Pointer to output handle");
            ITensor &t = Deref<ITensor>(TensorPool(), handle);
            if (rank < 1 || rank > NVCV_TENSOR_MAX_RANK)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Number of dimensions must be between 1 and %d, not %d",
                            NVCV_TENSOR_MAX_RANK, rank);
            }
            NotNull(shape, "Pointer to shape");
            if (layout.rank > 0 && layout.rank != rank)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT,
                            "The number of dimensions of the provided layout (%d) and shape (%d) do not match",
                            layout.rank, rank);
            }
            NVCVTensorData d;
            t.exportData(d);
            int64_t oldVol = 1, newVol = 1;
            for (int i = 0; i < d.rank; ++i)
            {
                oldVol *= d.shape[i];
            }
            for (int i = 0; i < rank; ++i)
            {
                if (shape[i] < 1)
                {
                    throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Shape #%d must be >= 1, not %ld", i, (long)shape[i]);
                }
                newVol *= shape[i];
            }
            if (oldVol != newVol)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT,
                            "The volume (%ld) of the provided shape does not match the size of the array (%ld)",
                            (long)newVol, (long)oldVol);
            }
            NVCVTensorData nd = d;
            nd.rank           = rank;
            nd.layout         = layout;
            std::fill_n(nd.shape, NVCV_TENSOR_MAX_RANK, int64_t(0));
            std::fill_n(nd.buffer.strided.strides, NVCV_TENSOR_MAX_RANK, int64_t(0));
            std::copy_n(shape, rank, nd.shape);
            if (!ViewStrides(d.rank, d.shape, d.buffer.strided.strides, rank, shape, nd.buffer.strided.strides))
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Cannot reshape: the memory layout does not allow this view");
            }
            TensorPool().incRef(handle);
            try
            {
                *out_handle = MakeWrapped(
                    nd,
                    [](void *ctx, const NVCVTensorData *)
                    {
                        try
                        {
                            TensorPool().decRef(ctx);
                        }
                        catch (...)
                        {
                        }
                    },
                    handle);
            }
            catch (...)
            {
                TensorPool().decRef(handle);
                throw;
            }
        });
}
}
