/* Status codes and the per-thread last-error slot.
 * Replaces: src/nvcv/src/include/nvcv/Status.h:48-172 (codes 0..11 keep their order),
 * behaviour of src/nvcv/src/priv/Status.cpp:31-110. */
#ifndef NVCV_STATUS_H
#define NVCV_STATUS_H

#include "Export.h"

#include <stdarg.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C"
{
#endif

typedef enum
{
    NVCV_SUCCESS                    = 0,
    NVCV_ERROR_NOT_IMPLEMENTED      = 1,
    NVCV_ERROR_INVALID_ARGUMENT     = 2,
    NVCV_ERROR_INVALID_IMAGE_FORMAT = 3,
    NVCV_ERROR_INVALID_OPERATION    = 4,
    NVCV_ERROR_DEVICE               = 5,
    NVCV_ERROR_NOT_READY            = 6,
    NVCV_ERROR_OUT_OF_MEMORY        = 7,
    NVCV_ERROR_INTERNAL             = 8,
    NVCV_ERROR_NOT_COMPATIBLE       = 9,
    NVCV_ERROR_OVERFLOW             = 10,
    NVCV_ERROR_UNDERFLOW            = 11
} NVCVStatus;

/* Size of the per-thread message buffer, terminating NUL included. */
#define NVCV_MAX_STATUS_MESSAGE_LENGTH (256)

/* Enumerator spelling of a status code, e.g. "NVCV_ERROR_OVERFLOW". */
NVCV_PUBLIC const char *nvcvStatusGetName(NVCVStatus code);

/* Read the calling thread's last status; GetLast* also resets it to NVCV_SUCCESS, Peek* does not.
 * The message variants copy at most lenBuffer bytes (always NUL-terminated) into msgBuffer. */
NVCV_PUBLIC NVCVStatus nvcvGetLastError(void);
NVCV_PUBLIC NVCVStatus nvcvGetLastErrorMessage(char *msgBuffer, int32_t lenBuffer);
NVCV_PUBLIC NVCVStatus nvcvPeekAtLastError(void);
NVCV_PUBLIC NVCVStatus nvcvPeekAtLastErrorMessage(char *msgBuffer, int32_t lenBuffer);

/* Overwrite the calling thread's status; fmt may be NULL (the message then becomes the code name). */
NVCV_PUBLIC void nvcvSetThreadStatus(NVCVStatus status, const char *fmt, ...)
#if defined(__GNUC__)
    __attribute__((format(printf, 2, 3)))
#endif
    ;
NVCV_PUBLIC void nvcvSetThreadStatusVarArgList(NVCVStatus status, const char *fmt, va_list va);

#ifdef __cplusplus
}
#endif

#endif /* NVCV_STATUS_H */
