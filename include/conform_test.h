/*
 * Test-side device hooks for HIP.
 *
 * The reference's conformance harness (diopi_test) is device-agnostic: its
 * runtime stub allocates, copies and synchronises through a handful of hooks
 * that each backend supplies next to its operator library (reference:
 * diopi_test/diopi_stub/include/conform_test.h:28-43; the CUDA versions are
 * impl/torch/test/conform_test.cpp:27-83).  libdiopirt_hip.so defines them for
 * HIP, with the same names, arguments and meaning, so the file that a
 * maintainer adds as impl/<backend>/test/conform_test.cpp is this set.
 *
 * Unlike the CUDA versions, which print a failed runtime call and go on, these
 * return diopiErrorOccurred (device_malloc: NULL) and print the HIP error to
 * stderr.  Copies are asynchronous on the given stream; the host buffer of an
 * h2d / d2h copy must stay valid until the stream has been synchronised.
 */
#ifndef DIOPI_ROCM_INCLUDE_CONFORM_TEST_H_
#define DIOPI_ROCM_INCLUDE_CONFORM_TEST_H_

#include <diopi/diopirt.h>

#if defined(__cplusplus)
extern "C" {
#endif

/* device memory (conform_test.h:28-29) */
void* device_malloc(uint64_t bytes);
void device_free(void* ptr);

/* asynchronous copies on a stream made by device_make_stream (conform_test.h:30-32) */
diopiError_t device_memcpy_h2d_async(diopiStreamHandle_t stream, void* deviceDst, const void* hostSrc, uint64_t bytes);
diopiError_t device_memcpy_d2h_async(diopiStreamHandle_t stream, void* hostDst, const void* deviceSrc, uint64_t bytes);
diopiError_t device_memcpy_d2d_async(diopiStreamHandle_t stream, void* deviceDst, const void* deviceSrc, uint64_t bytes);

/* streams: a diopiStreamHandle_t made here is a hipStream_t at the default priority (conform_test.h:33-35) */
diopiError_t device_make_stream(diopiStreamHandle_t* stream);
diopiError_t device_destroy_stream(diopiStreamHandle_t stream);
diopiError_t device_synchronize_stream(diopiStreamHandle_t stream);

/* Nothing to set up or tear down: the operator library needs no init call (conform_test.h:40-41). */
diopiError_t initLibrary(void);
diopiError_t finalizeLibrary(void);

/* Makes `out` a host uint8 tensor of 808 bytes owned by `ctx`, the size of the state the reference hands to its
 * random-number operators (conform_test.h:43; impl/torch/test/conform_test.cpp:75-82).  No operator of this library
 * draws random numbers; the hook exists so that the harness links. */
diopiError_t buildGeneratorState(diopiContextHandle_t ctx, diopiTensorHandle_t out);

#if defined(__cplusplus)
}
#endif

#endif /* DIOPI_ROCM_INCLUDE_CONFORM_TEST_H_ */
