/*
 * Library identification entry points exported by libdiopi_impl.so.
 * reference: proto/include/diopi/functions.h:19-21.  The remaining ~400
 * prototypes of that header belong to other operator families and are left
 * undefined; consumers hold them as weak symbols and test the address first.
 */
#ifndef DIOPI_ROCM_INCLUDE_DIOPI_FUNCTIONS_H_
#define DIOPI_ROCM_INCLUDE_DIOPI_FUNCTIONS_H_

#include <diopi/diopirt.h>

#if defined(__cplusplus)
extern "C" {
#endif

/* Contains the substring "Device" (the harness asserts it); this library returns "RocmDevice". */
DIOPI_RT_API DIOPI_ATTR_WEAK const char* diopiGetVendorName();
/* "HIP Version: ...; DIOPI Version: 1.0.0; arch gfx950" */
DIOPI_RT_API DIOPI_ATTR_WEAK const char* diopiGetImplVersion();
/* Text of the most recent failure in this process: "hip error: <..>; other error: <..>".
 * The returned pointer stays valid; the buffer is guarded by a mutex. */
DIOPI_RT_API DIOPI_ATTR_WEAK const char* diopiGetLastErrorString();

#if defined(__cplusplus)
}
#endif

#endif /* DIOPI_ROCM_INCLUDE_DIOPI_FUNCTIONS_H_ */
