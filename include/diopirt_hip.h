/*
 * libdiopirt_hip.so: a small HIP-backed implementation of the caller side of
 * the DIOPI runtime interface (the callbacks declared in diopi/diopirt.h),
 * plus a plain-C control surface so that a ctypes / FFI harness can build
 * contexts and tensor handles without a C++ binding layer.
 *
 * It plays the role that diopi_test/diopi_stub/csrc/litert.cpp plays for the
 * reference (tensor + context objects at litert.hpp:81-156, 229-277; callbacks
 * at litert.cpp:209-330).  It is a test companion: a framework that already
 * implements diopirt.h links libdiopi_impl.so against its own runtime instead.
 *
 * Differences from the reference stub, on purpose:
 *  - tensors can *wrap* memory that somebody else owns (a torch tensor, a
 *    hipMalloc'ed block) instead of always owning a fresh allocation;
 *  - scratch obtained through diopiRequireTensor/diopiRequireBuffer comes from
 *    a per-context pool that is recycled by diopirtContextClearTensors, so a
 *    steady-state serving loop performs no hipMalloc/hipFree;
 *  - a context may adopt an existing hipStream_t.
 */
#ifndef DIOPI_ROCM_INCLUDE_DIOPIRT_HIP_H_
#define DIOPI_ROCM_INCLUDE_DIOPIRT_HIP_H_

#include <diopi/diopirt.h>

#if defined(__cplusplus)
extern "C" {
#endif

/* Number of HIP devices visible to the process (0 when there is none; never fails). */
int diopirtDeviceCount(void);

/* Maximum shader clock in kHz and number of compute units of a device (0 when the query fails). */
int diopirtDeviceClockKHz(int device);
int diopirtDeviceComputeUnits(int device);

/* Create a context.  `stream` is an existing hipStream_t to adopt, or NULL to
 * let the context create its own non-blocking stream on first use. */
diopiContextHandle_t diopirtContextCreate(void* stream);
/* Destroys the context, its own stream (if it created one) and its scratch pool. */
void diopirtContextDestroy(diopiContextHandle_t ctx);
/* Hands every tensor given out by diopiRequireTensor/Buffer back to the pool.
 * Does not synchronise: stream order keeps reuse safe on the context's stream. */
void diopirtContextClearTensors(diopiContextHandle_t ctx);
/* Blocks until all work queued on the context's stream has finished. */
diopiError_t diopirtContextSynchronize(diopiContextHandle_t ctx);
/* Bytes currently handed out / high-water mark of the scratch pool, number of hipMalloc calls so far. */
int64_t diopirtContextScratchInUse(diopiContextHandle_t ctx);
int64_t diopirtContextScratchPeak(diopiContextHandle_t ctx);
int64_t diopirtContextMallocCount(diopiContextHandle_t ctx);

/* Wrap caller-owned memory as a tensor handle.  `stride` may be NULL (contiguous).
 * The handle must be released with diopirtTensorDestroy; the memory is not touched. */
diopiTensorHandle_t diopirtTensorWrap(void* data, const int64_t* shape, const int64_t* stride, int64_t ndim, diopiDtype_t dtype, diopiDevice_t device);
void diopirtTensorDestroy(diopiTensorHandle_t th);

/* Timing on the context's own stream with HIP events. */
void* diopirtEventCreate(void);
void diopirtEventDestroy(void* ev);
diopiError_t diopirtEventRecord(void* ev, diopiContextHandle_t ctx);
/* Waits for `stop`, returns milliseconds between the two events (negative on error). */
float diopirtEventElapsedMs(void* start, void* stop);

/* Size in bytes of one element of `dtype` (0 for unsupported). */
int64_t diopirtItemsize(diopiDtype_t dtype);

#if defined(__cplusplus)
}
#endif

#endif /* DIOPI_ROCM_INCLUDE_DIOPIRT_HIP_H_ */
