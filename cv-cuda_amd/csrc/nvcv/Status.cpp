// Per-thread status slot and the status entry points.
// Behaviour follows src/nvcv/src/priv/Status.cpp:31-110 and src/nvcv/src/Status.cpp of the reference.
#include "Priv.hpp"

#include <cstring>

namespace nvcvamd {

namespace {
struct ThreadStatus
{
    NVCVStatus code = NVCV_SUCCESS;
    char       msg[NVCV_MAX_STATUS_MESSAGE_LENGTH] = "success";
};

ThreadStatus &Slot() noexcept
{
    static thread_local ThreadStatus s;
    return s;
}
} // namespace

Error::Error(NVCVStatus code, const char *fmt, ...)
    : m_code(code)
{
    va_list va;
    va_start(va, fmt);
    vsnprintf(m_msg, sizeof(m_msg), fmt, va);
    va_end(va);
}

void SetThreadStatus(NVCVStatus code, const char *msg) noexcept
{
    ThreadStatus &s = Slot();
    s.code          = code;
    snprintf(s.msg, sizeof(s.msg), "%s", msg ? msg : nvcvStatusGetName(code));
}

void SetThreadStatusFromCurrentException() noexcept
{
    try
    {
        throw;
    }
    catch (const Error &e)
    {
        SetThreadStatus(e.code(), e.what());
    }
    catch (const std::invalid_argument &e)
    {
        SetThreadStatus(NVCV_ERROR_INVALID_ARGUMENT, e.what());
    }
    catch (const std::bad_alloc &)
    {
        SetThreadStatus(NVCV_ERROR_OUT_OF_MEMORY, "Not enough space for resource allocation");
    }
    catch (const std::exception &e)
    {
        SetThreadStatus(NVCV_ERROR_INTERNAL, e.what());
    }
    catch (...)
    {
        SetThreadStatus(NVCV_ERROR_INTERNAL, "Unexpected error");
    }
}

NVCVStatus PeekThreadStatus(char *msg, int32_t len) noexcept
{
    ThreadStatus &s = Slot();
    if (msg != nullptr && len > 0)
    {
        snprintf(msg, (size_t)len, "%s", s.msg);
    }
    return s.code;
}

} // namespace nvcvamd

using namespace nvcvamd;

extern "C"
{
const char *nvcvStatusGetName(NVCVStatus code)
{
    switch (EnumValue(code))
    {
#define NAME(x) \
    case x:     \
        return #x
        NAME(NVCV_SUCCESS);
        NAME(NVCV_ERROR_NOT_IMPLEMENTED);
        NAME(NVCV_ERROR_INVALID_ARGUMENT);
        NAME(NVCV_ERROR_INVALID_IMAGE_FORMAT);
        NAME(NVCV_ERROR_INVALID_OPERATION);
        NAME(NVCV_ERROR_DEVICE);
        NAME(NVCV_ERROR_NOT_READY);
        NAME(NVCV_ERROR_OUT_OF_MEMORY);
        NAME(NVCV_ERROR_INTERNAL);
        NAME(NVCV_ERROR_NOT_COMPATIBLE);
        NAME(NVCV_ERROR_OVERFLOW);
        NAME(NVCV_ERROR_UNDERFLOW);
#undef NAME
    }
    return "Unknown error";
}

NVCVStatus nvcvPeekAtLastError(void)
{
    return PeekThreadStatus(nullptr, 0);
}

NVCVStatus nvcvPeekAtLastErrorMessage(char *msgBuffer, int32_t lenBuffer)
{
    return PeekThreadStatus(msgBuffer, lenBuffer);
}

NVCVStatus nvcvGetLastError(void)
{
    return nvcvGetLastErrorMessage(nullptr, 0);
}

NVCVStatus nvcvGetLastErrorMessage(char *msgBuffer, int32_t lenBuffer)
{
    NVCVStatus st = PeekThreadStatus(msgBuffer, lenBuffer);
    SetThreadStatus(NVCV_SUCCESS, "success");
    return st;
}

void nvcvSetThreadStatusVarArgList(NVCVStatus status, const char *fmt, va_list va)
{
    if (fmt == nullptr)
    {
        SetThreadStatus(status, ""); // no message given: the message is empty, not the status name
        return;
    }
    char buf[NVCV_MAX_STATUS_MESSAGE_LENGTH];
    vsnprintf(buf, sizeof(buf), fmt, va);
    SetThreadStatus(status, buf);
}

void nvcvSetThreadStatus(NVCVStatus status, const char *fmt, ...)
{
    va_list va;
    va_start(va, fmt);
    nvcvSetThreadStatusVarArgList(status, fmt, va);
    va_end(va);
}
}
