/* Operator handles. Replaces: src/cvcuda/include/cvcuda/Operator.h:28-36 and detail/Export.h. */
#ifndef CVCUDA_OPERATOR_H
#define CVCUDA_OPERATOR_H

#if defined(__GNUC__)
#    define CVCUDA_PUBLIC __attribute__((visibility("default")))
#else
#    define CVCUDA_PUBLIC
#endif

#ifdef __cplusplus
extern "C"
{
#endif

typedef struct NVCVOperator *NVCVOperatorHandle;

/* Frees an operator made by any cvcuda*Create. NULL is ignored. Work already submitted keeps
 * running; operator-owned device buffers are released after the device has drained them. */
CVCUDA_PUBLIC void nvcvOperatorDestroy(NVCVOperatorHandle handle);

#ifdef __cplusplus
}
#endif

#endif /* CVCUDA_OPERATOR_H */
