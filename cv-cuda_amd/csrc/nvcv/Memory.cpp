// Memory requirements arithmetic, allocator objects and the handle pools.
// Requirements: src/nvcv/src/priv/Requirements.cpp:49-109. Default allocator:
// src/nvcv/src/priv/DefaultAllocator.cpp:29-84, on the HIP runtime (hipMalloc / hipHostMalloc).
// Handle pools: external behaviour of src/nvcv/src/priv/HandleManagerImpl.hpp:251-439.
#include "Priv.hpp"

#include <hip/hip_runtime_api.h>

#include <cstdlib>
#include <cstring>
#include <limits>

namespace nvcvamd {

// ---- requirements --------------------------------------------------------------------------------
void ReqAddBuffer(NVCVMemRequirements &m, int64_t size, int64_t align)
{
    if (align <= 0 || !IsPow2(align))
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Buffer alignment must be a power of two > 0, not %ld", (long)align);
    }
    int lg = ILog2(align);
    if (lg >= NVCV_MAX_MEM_REQUIREMENTS_LOG2_BLOCK_SIZE)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Buffer alignment must be < %ld, not %ld",
                    (long)NVCV_MAX_MEM_REQUIREMENTS_BLOCK_SIZE, (long)align);
    }
    int64_t mag    = size < 0 ? -size : size;
    int64_t blocks = (mag + align - 1) >> lg;
    if (size >= 0)
    {
        if (m.numBlocks[lg] > std::numeric_limits<int64_t>::max() - blocks)
        {
            throw Error(NVCV_ERROR_OVERFLOW, "Number of blocks with alignment %ld would overflow", (long)align);
        }
        m.numBlocks[lg] += blocks;
    }
    else
    {
        m.numBlocks[lg] = m.numBlocks[lg] > blocks ? m.numBlocks[lg] - blocks : 0;
    }
}

int64_t ReqTotalBytes(const NVCVMemRequirements &m)
{
    unsigned __int128 total = 0;
    for (int i = 0; i < NVCV_MAX_MEM_REQUIREMENTS_LOG2_BLOCK_SIZE; ++i)
    {
        total += (unsigned __int128)(uint64_t)m.numBlocks[i] << i;
    }
    if (total > (unsigned __int128)std::numeric_limits<int64_t>::max())
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Memory size overflow");
    }
    return (int64_t)total;
}

// ---- handle pools --------------------------------------------------------------------------------
HandlePool::HandlePool(const char *name)
    : m_name(name)
{
}

HandlePool::~HandlePool()
{
    // Process teardown. Live objects are reported (NVCV_LEAK_DETECTION=warn|abort) but not destroyed:
    // the HIP runtime may already be gone and destructors would call into it.
    int live = m_live.load();
    if (live > 0)
    {
        const char *mode = std::getenv("NVCV_LEAK_DETECTION");
        if (mode != nullptr && (std::strcmp(mode, "warn") == 0 || std::strcmp(mode, "abort") == 0))
        {
            std::fprintf(stderr, "nvcv: %d %s handle(s) were never destroyed\n", live, m_name);
            if (std::strcmp(mode, "abort") == 0)
            {
                std::abort();
            }
        }
    }
    for (int i = 0; i < m_numSlabs.load(); ++i)
    {
        ::operator delete[](m_slabs[i], std::align_val_t(alignof(HandleSlot)));
    }
}

void HandlePool::addSlab(int count)
{
    int n = m_numSlabs.load();
    if (n >= kMaxSlabs)
    {
        throw Error(NVCV_ERROR_OUT_OF_MEMORY, "Too many %s handles", m_name);
    }
    void       *mem  = ::operator new[](sizeof(HandleSlot) * (size_t)count, std::align_val_t(alignof(HandleSlot)));
    HandleSlot *slab = static_cast<HandleSlot *>(mem);
    for (int i = 0; i < count; ++i)
    {
        new (&slab[i]) HandleSlot();
        slab[i].nextFree = m_free;
        m_free           = &slab[i];
    }
    m_slabs[n]     = slab;
    m_slabCount[n] = count;
    m_capacity += count;
    m_numSlabs.store(n + 1, std::memory_order_release);
}

void *HandlePool::create(std::unique_ptr<CoreObject> obj)
{
    std::lock_guard<std::mutex> lock(m_mtx);
    // a fixed size caps the live objects also where the pool had grown beyond it before
    if (m_fixed && m_live.load() >= m_limit)
    {
        throw Error(NVCV_ERROR_OUT_OF_MEMORY, "%s handle pool is full (fixed capacity %d)", m_name, m_limit);
    }
    if (m_free == nullptr)
    {
        addSlab(m_capacity == 0 ? 256 : m_capacity);
    }
    HandleSlot *s = m_free;
    m_free        = s->nextFree;
    s->nextFree   = nullptr;
    s->refs.store(1);
    s->obj.store(obj.release(), std::memory_order_release);
    m_live.fetch_add(1);
    return reinterpret_cast<void *>(reinterpret_cast<uintptr_t>(s) | (s->generation.load() & 0xF));
}

HandleSlot *HandlePool::slotOf(void *handle) const
{
    if (handle == nullptr)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "%s handle cannot be NULL", m_name);
    }
    uintptr_t   raw  = reinterpret_cast<uintptr_t>(handle);
    uintptr_t   addr = raw & ~uintptr_t(0xF);
    HandleSlot *slot = nullptr;
    int         n    = m_numSlabs.load(std::memory_order_acquire);
    for (int i = 0; i < n; ++i)
    {
        uintptr_t base = reinterpret_cast<uintptr_t>(m_slabs[i]);
        if (addr >= base && addr < base + sizeof(HandleSlot) * (size_t)m_slabCount[i]
            && (addr - base) % sizeof(HandleSlot) == 0)
        {
            slot = reinterpret_cast<HandleSlot *>(addr);
            break;
        }
    }
    if (slot == nullptr || slot->obj.load(std::memory_order_acquire) == nullptr
        || (slot->generation.load() & 0xF) != (raw & 0xF))
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "The %s handle is invalid or was already destroyed", m_name);
    }
    return slot;
}

CoreObject *HandlePool::get(void *handle) const
{
    return slotOf(handle)->obj.load(std::memory_order_acquire);
}

int HandlePool::incRef(void *handle)
{
    return slotOf(handle)->refs.fetch_add(1) + 1;
}

int HandlePool::refCount(void *handle) const
{
    return slotOf(handle)->refs.load();
}

int HandlePool::decRef(void *handle)
{
    HandleSlot *s    = slotOf(handle);
    int         left = s->refs.fetch_sub(1) - 1;
    if (left == 0)
    {
        CoreObject *obj = s->obj.exchange(nullptr);
        s->generation.fetch_add(1);
        delete obj; // may release further handles (allocator, wrapped image)
        std::lock_guard<std::mutex> lock(m_mtx);
        s->nextFree = m_free;
        m_free      = s;
        m_live.fetch_sub(1);
    }
    return left;
}

void HandlePool::setFixedSize(int32_t maxCount)
{
    std::lock_guard<std::mutex> lock(m_mtx);
    if (maxCount < 0)
    {
        m_fixed = false;
        return;
    }
    if (m_live.load() > 0)
    {
        throw Error(NVCV_ERROR_INVALID_OPERATION, "Cannot change the size policy while there are still %d live %s handles",
                    m_live.load(), m_name);
    }
    if (m_capacity < maxCount)
    {
        addSlab(maxCount - m_capacity);
    }
    m_fixed = true;
    m_limit = maxCount;
}

HandlePool &AllocatorPool()
{
    static HandlePool *p = new HandlePool("allocator"); // intentionally outlives static destructors of users
    return *p;
}

HandlePool &TensorPool()
{
    static HandlePool *p = new HandlePool("tensor");
    return *p;
}

HandlePool &ImagePool()
{
    static HandlePool *p = new HandlePool("image");
    return *p;
}

HandlePool &ImageBatchPool()
{
    static HandlePool *p = new HandlePool("image batch");
    return *p;
}

// ---- allocators ----------------------------------------------------------------------------------
namespace {

void CheckAllocArgs(int64_t size, int32_t align)
{
    if (size < 0)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Allocation size must be >= 0, not %ld", (long)size);
    }
    if (!IsPow2(align))
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Alignment must be a power of two, not %d", align);
    }
    // reference: src/nvcv/src/priv/IAllocator.cpp:45-50, a size that is not whole alignment units is rejected
    if (AlignUp(size, (int64_t)align) != size)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Allocation size must be an integral multiple of alignment %d, not %ld",
                    align, (long)size);
    }
}

void *DefaultAllocHost(void *, int64_t size, int32_t align)
{
    size_t a = (size_t)std::max<int32_t>(align, (int32_t)sizeof(void *));
    return std::aligned_alloc(a, (size_t)AlignUp(std::max<int64_t>(size, 1), (int64_t)a));
}

void DefaultFreeHost(void *, void *p, int64_t, int32_t)
{
    std::free(p);
}

void *DefaultAllocPinned(void *, int64_t size, int32_t)
{
    void *p = nullptr;
    if (hipHostMalloc(&p, (size_t)std::max<int64_t>(size, 1), hipHostMallocDefault) != hipSuccess)
    {
        (void)hipGetLastError();
        return nullptr;
    }
    return p;
}

void DefaultFreePinned(void *, void *p, int64_t, int32_t)
{
    if (p != nullptr)
    {
        (void)hipHostFree(p);
    }
}

void *DefaultAllocDevice(void *, int64_t size, int32_t)
{
    // hipMalloc returns at least 256-byte aligned addresses; larger requests come back page aligned.
    void *p = nullptr;
    if (hipMalloc(&p, (size_t)std::max<int64_t>(size, 1)) != hipSuccess)
    {
        (void)hipGetLastError();
        return nullptr;
    }
    return p;
}

void DefaultFreeDevice(void *, void *p, int64_t, int32_t)
{
    if (p != nullptr)
    {
        (void)hipFree(p);
    }
}

class Allocator final : public IAllocator
{
public:
    Allocator()
    {
        m_res[NVCV_RESOURCE_MEM_HOST]        = {nullptr, NVCV_RESOURCE_MEM_HOST, {{DefaultAllocHost, DefaultFreeHost}}, nullptr};
        m_res[NVCV_RESOURCE_MEM_CUDA]        = {nullptr, NVCV_RESOURCE_MEM_CUDA, {{DefaultAllocDevice, DefaultFreeDevice}}, nullptr};
        m_res[NVCV_RESOURCE_MEM_HOST_PINNED] = {nullptr, NVCV_RESOURCE_MEM_HOST_PINNED, {{DefaultAllocPinned, DefaultFreePinned}}, nullptr};
    }

    Allocator(const NVCVResourceAllocator *custom, int32_t n)
        : Allocator()
    {
        // Validate everything before taking ownership of any entry: if construction fails the
        // caller keeps its contexts and no cleanup callback must run.
        bool seen[NVCV_NUM_RESOURCE_TYPES] = {};
        for (int i = 0; i < n; ++i)
        {
            const NVCVResourceAllocator &c = custom[i];
            if ((int)c.resType < 0 || (int)c.resType >= NVCV_NUM_RESOURCE_TYPES)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Invalid resource type %d", (int)c.resType);
            }
            if (seen[c.resType])
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Custom memory allocator for %s is already defined",
                            nvcvResourceTypeGetName(c.resType));
            }
            if (c.res.mem.fnAlloc == nullptr || c.res.mem.fnFree == nullptr)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Custom allocation and deallocation functions must not be NULL");
            }
            seen[c.resType] = true;
        }
        for (int i = 0; i < n; ++i)
        {
            m_res[custom[i].resType] = custom[i];
        }
    }

    ~Allocator() override
    {
        for (NVCVResourceAllocator &r : m_res)
        {
            if (r.cleanup != nullptr)
            {
                r.cleanup(r.ctx, &r);
            }
        }
    }

    void *allocHost(int64_t size, int32_t align) override
    {
        return doAlloc(NVCV_RESOURCE_MEM_HOST, size, align);
    }

    void freeHost(void *p, int64_t size, int32_t align) noexcept override
    {
        doFree(NVCV_RESOURCE_MEM_HOST, p, size, align);
    }

    void *allocPinned(int64_t size, int32_t align) override
    {
        return doAlloc(NVCV_RESOURCE_MEM_HOST_PINNED, size, align);
    }

    void freePinned(void *p, int64_t size, int32_t align) noexcept override
    {
        doFree(NVCV_RESOURCE_MEM_HOST_PINNED, p, size, align);
    }

    void *allocDevice(int64_t size, int32_t align) override
    {
        return doAlloc(NVCV_RESOURCE_MEM_CUDA, size, align);
    }

    void freeDevice(void *p, int64_t size, int32_t align) noexcept override
    {
        doFree(NVCV_RESOURCE_MEM_CUDA, p, size, align);
    }

    void get(NVCVResourceType type, NVCVResourceAllocator *out) override
    {
        if ((int)type < 0 || (int)type >= NVCV_NUM_RESOURCE_TYPES)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Invalid resource type %d", (int)type);
        }
        // The stored descriptor as given (reference: src/nvcv/src/priv/CustomAllocator.cpp:120-124). The context it
        // names stays owned by this object: the cleanup callback is for the owner to run, once.
        *out = m_res[type];
    }

private:
    void *doAlloc(NVCVResourceType t, int64_t size, int32_t align)
    {
        CheckAllocArgs(size, align);
        void *p = m_res[t].res.mem.fnAlloc(m_res[t].ctx, size, align);
        if (p == nullptr)
        {
            throw Error(NVCV_ERROR_OUT_OF_MEMORY, "Cannot allocate %ld bytes of %s", (long)size,
                        nvcvResourceTypeGetName(t));
        }
        if ((reinterpret_cast<uintptr_t>(p) & (uintptr_t)(align - 1)) != 0)
        {
            m_res[t].res.mem.fnFree(m_res[t].ctx, p, size, align);
            throw Error(NVCV_ERROR_INTERNAL, "%s allocator returned memory not aligned to %d bytes",
                        nvcvResourceTypeGetName(t), align);
        }
        return p;
    }

    void doFree(NVCVResourceType t, void *p, int64_t size, int32_t align) noexcept
    {
        if (p != nullptr)
        {
            m_res[t].res.mem.fnFree(m_res[t].ctx, p, size, align);
        }
    }

    NVCVResourceAllocator m_res[NVCV_NUM_RESOURCE_TYPES];
};

} // namespace

IAllocator &DefaultAllocator()
{
    static Allocator *a = new Allocator();
    return *a;
}

IAllocator &ResolveAllocator(NVCVAllocatorHandle h, NVCVAllocatorHandle *held)
{
    *held = nullptr;
    if (h == nullptr)
    {
        return DefaultAllocator();
    }
    IAllocator &a = Deref<IAllocator>(AllocatorPool(), h);
    AllocatorPool().incRef(h);
    *held = h;
    return a;
}

} // namespace nvcvamd

using namespace nvcvamd;

extern "C"
{
NVCVStatus nvcvRequirementsInit(NVCVRequirements *req)
{
    return Protect([&] { std::memset(NotNull(req, "Pointer to requirements"), 0, sizeof(*req)); });
}

NVCVStatus nvcvRequirementsAdd(NVCVRequirements *reqSum, const NVCVRequirements *req)
{
    return Protect(
        [&]
        {
            NotNull(reqSum, "Pointer to summed requirements");
            NotNull(req, "Pointer to requirements");
            for (int i = 0; i < NVCV_MAX_MEM_REQUIREMENTS_LOG2_BLOCK_SIZE; ++i)
            {
                reqSum->cudaMem.numBlocks[i] += req->cudaMem.numBlocks[i];
                reqSum->hostMem.numBlocks[i] += req->hostMem.numBlocks[i];
                reqSum->hostPinnedMem.numBlocks[i] += req->hostPinnedMem.numBlocks[i];
            }
        });
}

NVCVStatus nvcvMemRequirementsCalcTotalSizeBytes(const NVCVMemRequirements *memReq, int64_t *sizeBytes)
{
    return Protect([&]
                   { *NotNull(sizeBytes, "Pointer to output size") = ReqTotalBytes(*NotNull(memReq, "Pointer to requirements")); });
}

NVCVStatus nvcvMemRequirementsAddBuffer(NVCVMemRequirements *memReq, int64_t bufSize, int64_t bufAlignment)
{
    return Protect([&] { ReqAddBuffer(*NotNull(memReq, "Pointer to requirements"), bufSize, bufAlignment); });
}

NVCVStatus nvcvAllocatorConstructCustom(const NVCVResourceAllocator *customAllocators, int32_t numCustomAllocators,
                                        NVCVAllocatorHandle *handle)
{
    return Protect(
        [&]
        {
            NotNull(handle, "Pointer to output handle");
            if (numCustomAllocators < 0 || (numCustomAllocators > 0 && customAllocators == nullptr))
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Array of custom allocators must not be NULL");
            }
            *handle = static_cast<NVCVAllocatorHandle>(
                AllocatorPool().create(std::make_unique<Allocator>(customAllocators, numCustomAllocators)));
        });
}

NVCVStatus nvcvAllocatorDecRef(NVCVAllocatorHandle handle, int *newRefCount)
{
    return Protect(
        [&]
        {
            int n = AllocatorPool().decRef(handle);
            if (newRefCount)
            {
                *newRefCount = n;
            }
        });
}

NVCVStatus nvcvAllocatorIncRef(NVCVAllocatorHandle handle, int *newRefCount)
{
    return Protect(
        [&]
        {
            int n = AllocatorPool().incRef(handle);
            if (newRefCount)
            {
                *newRefCount = n;
            }
        });
}

NVCVStatus nvcvAllocatorRefCount(NVCVAllocatorHandle handle, int *newRefCount)
{
    return Protect([&] { *NotNull(newRefCount, "Pointer to output") = AllocatorPool().refCount(handle); });
}

NVCVStatus nvcvAllocatorGet(NVCVAllocatorHandle handle, NVCVResourceType resType, NVCVResourceAllocator *result)
{
    return Protect(
        [&]
        {
            NotNull(result, "Pointer to output");
            IAllocator &a = handle ? Deref<IAllocator>(AllocatorPool(), handle) : DefaultAllocator();
            a.get(resType, result);
        });
}

NVCVStatus nvcvAllocatorSetUserPointer(NVCVAllocatorHandle handle, void *userPtr)
{
    return Protect([&] { AllocatorPool().get(handle)->userPtr = userPtr; });
}

NVCVStatus nvcvAllocatorGetUserPointer(NVCVAllocatorHandle handle, void **outUserPtr)
{
    return Protect([&] { *NotNull(outUserPtr, "Pointer to output") = AllocatorPool().get(handle)->userPtr; });
}

#define NVCVAMD_ALLOC_PAIR(Name, allocFn, freeFn)                                                                  \
    NVCVStatus nvcvAllocatorAlloc##Name(NVCVAllocatorHandle halloc, void **ptr, int64_t sizeBytes, int32_t alignBytes) \
    {                                                                                                              \
        return Protect(                                                                                            \
            [&]                                                                                                    \
            {                                                                                                      \
                NotNull(ptr, "Pointer to output buffer");                                                          \
                IAllocator &a = halloc ? Deref<IAllocator>(AllocatorPool(), halloc) : DefaultAllocator();          \
                *ptr          = a.allocFn(sizeBytes, alignBytes);                                                  \
            });                                                                                                    \
    }                                                                                                              \
    NVCVStatus nvcvAllocatorFree##Name(NVCVAllocatorHandle halloc, void *ptr, int64_t sizeBytes, int32_t alignBytes) \
    {                                                                                                              \
        return Protect(                                                                                            \
            [&]                                                                                                    \
            {                                                                                                      \
                IAllocator &a = halloc ? Deref<IAllocator>(AllocatorPool(), halloc) : DefaultAllocator();          \
                a.freeFn(ptr, sizeBytes, alignBytes);                                                              \
            });                                                                                                    \
    }

NVCVAMD_ALLOC_PAIR(HostMemory, allocHost, freeHost)
NVCVAMD_ALLOC_PAIR(HostPinnedMemory, allocPinned, freePinned)
NVCVAMD_ALLOC_PAIR(CudaMemory, allocDevice, freeDevice)
#undef NVCVAMD_ALLOC_PAIR

const char *nvcvResourceTypeGetName(NVCVResourceType resource)
{
    switch (EnumValue(resource)) // callers may pass any integer
    {
    case NVCV_RESOURCE_MEM_HOST:
        return "NVCV_RESOURCE_MEM_HOST";
    case NVCV_RESOURCE_MEM_CUDA:
        return "NVCV_RESOURCE_MEM_CUDA";
    case NVCV_RESOURCE_MEM_HOST_PINNED:
        return "NVCV_RESOURCE_MEM_HOST_PINNED";
    }
    return "Unexpected error retrieving NVCVResourceType string representation";
}

NVCVStatus nvcvConfigSetMaxImageCount(int32_t maxCount)
{
    return Protect([&] { ImagePool().setFixedSize(maxCount); });
}

NVCVStatus nvcvConfigSetMaxImageBatchCount(int32_t maxCount)
{
    return Protect([&] { ImageBatchPool().setFixedSize(maxCount); });
}

NVCVStatus nvcvConfigSetMaxTensorCount(int32_t maxCount)
{
    return Protect([&] { TensorPool().setFixedSize(maxCount); });
}

NVCVStatus nvcvConfigSetMaxAllocatorCount(int32_t maxCount)
{
    return Protect([&] { AllocatorPool().setFixedSize(maxCount); });
}

NVCVStatus nvcvConfigSetMaxArrayCount(int32_t /*maxCount*/)
{
    // No array objects exist in this library, so there is no pool to size.
    return NVCV_SUCCESS;
}

uint32_t nvcvGetVersion(void)
{
    return NVCV_VERSION;
}
}
