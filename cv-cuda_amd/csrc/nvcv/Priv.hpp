// Internals shared by the NVCV core sources: error transport, integer helpers, format decoding,
// the handle pools and the object interfaces behind the C handles.
#ifndef NVCV_AMD_PRIV_HPP
#define NVCV_AMD_PRIV_HPP

#include <nvcv/Config.h>
#include <nvcv/ImageBatch.h>
#include <nvcv/Tensor.h>
#include <nvcv/TensorShape.h>
#include <nvcv/Version.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <exception>
#include <memory>
#include <mutex>
#include <new>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace nvcvamd {

// ---------------------------------------------------------------------------------------------
// Error transport: internal code throws Error; every C entry point runs inside Protect(), which
// stores {code, message} in the calling thread's slot and returns the code
// (same contract as the reference's ProtectCall, src/nvcv/src/priv/Status.hpp + Status.cpp:31-81).
class Error : public std::exception
{
public:
    Error(NVCVStatus code, const char *fmt, ...) __attribute__((format(printf, 3, 4)));

    NVCVStatus code() const noexcept
    {
        return m_code;
    }

    const char *what() const noexcept override
    {
        return m_msg;
    }

private:
    NVCVStatus m_code;
    char       m_msg[NVCV_MAX_STATUS_MESSAGE_LENGTH];
};

void       SetThreadStatus(NVCVStatus code, const char *msg) noexcept;
void       SetThreadStatusFromCurrentException() noexcept;
NVCVStatus PeekThreadStatus(char *msg, int32_t len) noexcept;

template<class F>
NVCVStatus Protect(F &&fn) noexcept
{
    try
    {
        fn();
        return NVCV_SUCCESS;
    }
    catch (...)
    {
        SetThreadStatusFromCurrentException();
        return PeekThreadStatus(nullptr, 0);
    }
}

// The value of an enumeration argument as an int, read through its bytes: C callers may pass any integer where
// the API names an enum, and reading a value outside the enumerators' range through the enum type is undefined.
template<class E>
inline int EnumValue(const E &e)
{
    static_assert(sizeof(E) == sizeof(int), "C enums of this API are int-sized");
    int v;
    __builtin_memcpy(&v, &e, sizeof(v));
    return v;
}

template<class T>
T *NotNull(T *p, const char *what)
{
    if (p == nullptr)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "%s must not be NULL", what);
    }
    return p;
}

// ---------------------------------------------------------------------------------------------
// Integer helpers
inline bool IsPow2(int64_t v)
{
    return v > 0 && (v & (v - 1)) == 0;
}

inline int64_t NextPow2(int64_t v)
{
    int64_t p = 1;
    while (p < v)
    {
        p <<= 1;
    }
    return p;
}

inline int64_t AlignUp(int64_t v, int64_t pow2)
{
    return (v + pow2 - 1) & ~(pow2 - 1);
}

inline int ILog2(int64_t pow2)
{
    int n = 0;
    while ((int64_t(1) << n) < pow2)
    {
        ++n;
    }
    return n;
}

// Default alignments of library-allocated buffers. 128 B is one gfx950 L2 cache line, so every
// row of a tensor or image starts on a line and a wavefront's 16-byte-per-lane accesses never
// straddle lines needlessly; 512 B keeps buffer starts aligned for any vector width.
constexpr int32_t kDefaultRowAlign  = 128;
constexpr int32_t kDefaultBaseAlign = 512;

// ---------------------------------------------------------------------------------------------
// Format decoding (Format.cpp)
struct PackingInfo
{
    int     numComponents; // values stored per pixel (group) in the plane (0 = plane absent)
    int     numChannels;   // image channels they carry: the same, except 3 for the 4:2:2 pixel-pair packings
    int     bitsPerPixel;  // storage bits per pixel
    int32_t bits[4];       // bits of each component, 0-terminated
    bool    known;         // false -> packing value not in the table
};

// One row of PackingTable.inc.
struct PackingRow
{
    NVCVPacking   packing;
    const char   *name;
    NVCVByteOrder order;
    int32_t       alignment;
    NVCVSwizzle   swizzle;   // positions of the channels among the stored fields; 0000 = fields are the channels
    int32_t       fields[4]; // widths of the stored fields in memory order, padding included
    int32_t       bits[4];   // widths of channels X, Y, Z, W
};
const PackingRow *FindPacking(NVCVPacking p);  // nullptr when the value is not a known packing
const PackingRow *PackingTable(int *count);

inline uint64_t FieldGet(uint64_t v, int off, int len)
{
    return NVCV_DETAIL_BITS_GET(v, off, len);
}

inline uint64_t FieldPut(uint64_t v, int off, int len)
{
    return NVCV_DETAIL_BITS_PUT(v, off, len);
}

// printf into one of a few per-thread buffers; the result stays valid for the next three calls of the thread.
const char *ThreadName(const char *fmt, ...);
// names[v] for v in [0,count), otherwise "<type>(<v>)".
const char *EnumName(int v, const char *const *names, int count, const char *type);

PackingInfo           DecodePacking(NVCVPacking p);
NVCVPacking           FormatPlanePacking(uint64_t fmt, int plane); // plane in [0,4)
int                   FormatNumPlanes(uint64_t fmt);
int                   FormatNumChannels(uint64_t fmt);
NVCVSwizzle           FormatSwizzle(uint64_t fmt);
NVCVDataKind          FormatDataKind(uint64_t fmt);
NVCVMemLayout         FormatMemLayout(uint64_t fmt);
NVCVColorModel        FormatColorModel(uint64_t fmt);
NVCVColorSpec         FormatColorSpec(uint64_t fmt);
NVCVChromaSubsampling FormatCSS(uint64_t fmt);
int                   FormatPlanePixelStrideBytes(uint64_t fmt, int plane);
NVCVDataType          FormatPlaneDataType(uint64_t fmt, int plane);
void                  FormatPlaneSize(uint64_t fmt, int plane, int32_t w, int32_t h, int32_t *pw, int32_t *ph);
void                  SwizzleChannels(NVCVSwizzle sw, NVCVChannel out[4]);
int                   SwizzleNumChannels(NVCVSwizzle sw);
uint64_t              MakeFormatWord(NVCVColorModel model, uint32_t specOrRaw, NVCVChromaSubsampling css,
                                     NVCVMemLayout layout, NVCVDataKind kind, NVCVSwizzle swizzle, NVCVAlphaType alpha,
                                     NVCVPacking p0, NVCVPacking p1, NVCVPacking p2, NVCVPacking p3,
                                     const NVCVExtraChannelInfo *ex = nullptr);
NVCVAlphaType         FormatAlphaType(uint64_t fmt);
NVCVExtraChannelInfo  FormatExtraChannels(uint64_t fmt);
int                   FormatRawPattern(uint64_t fmt); // -1 when the colour model is not RAW
NVCVSwizzle           MakeSwizzle(NVCVChannel x, NVCVChannel y, NVCVChannel z, NVCVChannel w); // UNSUPPORTED if not in the table
// Validating constructor behind every nvcvMake*ImageFormat entry point and the setters that rebuild a format.
uint64_t MakeCheckedFormat(NVCVColorModel model, uint32_t specOrRaw, NVCVChromaSubsampling css, NVCVMemLayout layout,
                           NVCVDataKind kind, NVCVSwizzle swizzle, NVCVPacking p0, NVCVPacking p1, NVCVPacking p2,
                           NVCVPacking p3, NVCVAlphaType alpha, const NVCVExtraChannelInfo *ex);

inline NVCVPacking DataTypePacking(NVCVDataType t)
{
    return FormatPlanePacking(t, 0);
}

int DataTypeStrideBytes(NVCVDataType t); // bytes per element, all channels
int DataTypeAlignment(NVCVDataType t);   // natural alignment of one element

// Layout helpers (Layout.cpp)
NVCVTensorLayout MakeLayout(const char *descr);
NVCVTensorLayout LayoutLast(const NVCVTensorLayout &l, int n);
inline bool      LayoutEq(const NVCVTensorLayout &a, const NVCVTensorLayout &b)
{
    return nvcvTensorLayoutCompare(a, b) == 0;
}
void PermuteShape(const NVCVTensorLayout &srcL, const int64_t *src, const NVCVTensorLayout &dstL, int64_t *dst);

// Requirements helpers (Memory.cpp)
void    ReqAddBuffer(NVCVMemRequirements &m, int64_t size, int64_t align);
int64_t ReqTotalBytes(const NVCVMemRequirements &m);

// ---------------------------------------------------------------------------------------------
// Core objects and handle pools.
//
// A handle is the address of a 16-byte-aligned pool slot with the slot's 4-bit generation in the
// low bits; freeing a slot bumps its generation so stale handles are detected instead of
// dereferenced (external behaviour of the reference's HandleManager,
// src/nvcv/src/priv/HandleManager.hpp:52-200, HandleManagerImpl.hpp:251-439).
class CoreObject
{
public:
    virtual ~CoreObject() = default;
    void *userPtr = nullptr;
};

struct alignas(16) HandleSlot
{
    std::atomic<CoreObject *> obj{nullptr};
    std::atomic<int>          refs{0};
    std::atomic<uint8_t>      generation{0};
    HandleSlot               *nextFree = nullptr;
};

class HandlePool
{
public:
    explicit HandlePool(const char *name);
    ~HandlePool();

    void *create(std::unique_ptr<CoreObject> obj); // refcount 1
    // Throws INVALID_ARGUMENT for NULL, foreign or stale handles.
    CoreObject *get(void *handle) const;
    int         incRef(void *handle);
    int         decRef(void *handle); // destroys the object when the count reaches 0
    int         refCount(void *handle) const;

    void setFixedSize(int32_t maxCount); // maxCount < 0 -> grow on demand
    int  liveCount() const
    {
        return m_live.load();
    }

private:
    HandleSlot *slotOf(void *handle) const;
    void        addSlab(int count);

    static constexpr int kMaxSlabs = 40;

    const char              *m_name;
    mutable std::mutex       m_mtx;
    HandleSlot              *m_free = nullptr;
    std::atomic<int>         m_numSlabs{0};
    HandleSlot              *m_slabs[kMaxSlabs]     = {};
    int                      m_slabCount[kMaxSlabs] = {};
    int                      m_capacity             = 0;
    bool                     m_fixed                = false;
    int                      m_limit                = 0; // live objects allowed while m_fixed
    std::atomic<int>         m_live{0};
};

HandlePool &AllocatorPool();
HandlePool &TensorPool();
HandlePool &ImagePool();
HandlePool &ImageBatchPool();

template<class T>
T &Deref(HandlePool &pool, void *handle)
{
    CoreObject *o = pool.get(handle);
    T          *t = dynamic_cast<T *>(o);
    if (t == nullptr)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Handle does not refer to an object of the expected type");
    }
    return *t;
}

// ---------------------------------------------------------------------------------------------
// Allocator objects (Memory.cpp). A null handle means the process-wide default allocator.
class IAllocator : public CoreObject
{
public:
    virtual void *allocHost(int64_t size, int32_t align)                  = 0;
    virtual void  freeHost(void *p, int64_t size, int32_t align) noexcept = 0;
    virtual void *allocPinned(int64_t size, int32_t align)                  = 0;
    virtual void  freePinned(void *p, int64_t size, int32_t align) noexcept = 0;
    virtual void *allocDevice(int64_t size, int32_t align)                  = 0;
    virtual void  freeDevice(void *p, int64_t size, int32_t align) noexcept = 0;
    virtual void  get(NVCVResourceType type, NVCVResourceAllocator *out)    = 0;
};

IAllocator &DefaultAllocator();

// Resolves a possibly-null allocator handle; for a non-null handle a reference is taken and
// returned in *held (to be released with AllocatorPool().decRef when the owner dies).
IAllocator &ResolveAllocator(NVCVAllocatorHandle h, NVCVAllocatorHandle *held);

class ITensor : public CoreObject
{
public:
    virtual void                exportData(NVCVTensorData &out) const = 0;
    virtual NVCVAllocatorHandle allocHandle() const                   = 0;
};

class IImage : public CoreObject
{
public:
    virtual NVCVTypeImage       type() const                         = 0;
    virtual void                size(int32_t *w, int32_t *h) const   = 0;
    virtual NVCVImageFormat     format() const                       = 0;
    virtual void                exportData(NVCVImageData &out) const = 0;
    virtual NVCVAllocatorHandle allocHandle() const                  = 0;
};

void ValidateWrappedTensor(const NVCVTensorData &d);

} // namespace nvcvamd

#endif // NVCV_AMD_PRIV_HPP
