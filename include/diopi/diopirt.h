/*
 * DIOPI runtime interface, restated for the gfx950 operator library.
 *
 * This header carries the part of the DIOPI C ABI that the operator library
 * and its caller share: value types, opaque handles and the callbacks the
 * library imports from whoever owns the tensors.  Only what the LLaMA inference
 * operators touch is restated; every declaration that is here is binary- and
 * source-compatible with the reference header (reference:
 * proto/include/diopi/diopirt.h, line numbers cited per block), so the
 * operators' translation units compile against either header directory.  The
 * scalar, memory-format, reduction and rounding-mode types of the reference
 * header (diopirt.h:81-96) have no user on this path and are left out.
 *
 * Direction of the calls:
 *   caller  --diopiXxx(ctx, tensors...)-->  operator library (functions_ext.h)
 *   caller  <--diopiGetTensorXxx, diopiGetStream, diopiRequireXxx--  operator library
 * The library never defines the callbacks; they are resolved against the
 * process that loaded it.
 */
#ifndef DIOPI_ROCM_INCLUDE_DIOPI_DIOPIRT_H_
#define DIOPI_ROCM_INCLUDE_DIOPI_DIOPIRT_H_

#include <stddef.h>
#include <stdint.h>

/* reference: diopirt.h:12-15 */
#define DIOPI_ATTR_WEAK __attribute__((weak))
#define DIOPI_API DIOPI_ATTR_WEAK
#define DIOPI_RT_API

#if defined(__cplusplus)
extern "C" {
#endif

/* interface version this library reports (reference: diopirt.h:22-24) */
#define DIOPI_VER_MAJOR 1
#define DIOPI_VER_MINOR 0
#define DIOPI_VER_PATCH 0

/* A borrowed array of int64 (shapes, strides, normalized_shape).  Passed by
 * value; the pointee stays owned by whoever produced it.  reference: diopirt.h:27-30 */
typedef struct {
    const int64_t* data;
    int64_t len;
} diopiSize_t;

/* Status codes.  0 is success; 13 tells the conformance harness to skip the
 * case; any other value is a hard failure whose text is diopiGetLastErrorString().
 * reference: diopirt.h:32-49 */
typedef enum {
    diopiSuccess = 0, diopiErrorOccurred = 1, diopiNotInited = 2,
    diopiNoRegisteredStreamCreateFunction = 3, diopiNoRegisteredStreamDestoryFunction = 4,
    diopiNoRegisteredStreamSyncFunction = 5, diopiNoRegisteredDeviceMemoryMallocFunction = 6,
    diopiNoRegisteredDeviceMemoryFreeFunction = 7, diopiNoRegisteredDevice2DdeviceMemoryCopyFunction = 8,
    diopiNoRegisteredDevice2HostMemoryCopyFunction = 9, diopiNoRegisteredHost2DeviceMemoryCopyFunction = 10,
    diopiNoRegisteredGetLastErrorFunction = 11, diopi5DNotSupported = 12,
    diopiNoImplement = 13, diopiForceFallbackToCPU = 14,
    diopiDtypeNotSupported = 1000,
} diopiError_t;

/* reference: diopirt.h:51-56 */
typedef enum { diopi_host = 0, diopi_device = 1 } diopiDevice_t;
typedef int8_t diopiDeviceIndex_t;

/* Element types; numeric values are part of the ABI.  reference: diopirt.h:60-79 */
typedef enum {
    diopi_dtype_int8 = 0, diopi_dtype_uint8 = 1, diopi_dtype_int16 = 2, diopi_dtype_uint16 = 3,
    diopi_dtype_int32 = 4, diopi_dtype_uint32 = 5, diopi_dtype_int64 = 6, diopi_dtype_uint64 = 7,
    diopi_dtype_float16 = 8, diopi_dtype_float32 = 9, diopi_dtype_float64 = 10,
    diopi_dtype_bool = 11, diopi_dtype_bfloat16 = 12, diopi_dtype_tfloat32 = 13,
    diopi_dtype_complex32 = 14, diopi_dtype_complex64 = 15, diopi_dtype_complex128 = 16,
    diopi_dtype_unsupported = 255
} diopiDtype_t;

/* Opaque handles: the library only ever passes them back to the callbacks.
 * reference: diopirt.h:98-112 */
struct diopiContext;
typedef struct diopiContext* diopiContextHandle_t;
struct diopiTensor;
typedef struct diopiTensor* diopiTensorHandle_t;
typedef const struct diopiTensor* diopiConstTensorHandle_t;
struct diopiGenerator;
typedef struct diopiGenerator* diopiGeneratorHandle_t;
typedef const struct diopiGenerator* diopiConstGeneratorHandle_t;
/* The native stream of the device runtime; here a hipStream_t. */
typedef void* diopiStreamHandle_t;

/* ---- tensor accessors, implemented by the caller (reference: diopirt.h:122-140) ----
 * The data pointer already includes any storage offset.  Shape and stride come
 * back as borrowed arrays that live as long as the tensor. */
diopiError_t diopiGetTensorData(diopiTensorHandle_t tensor, void** data);
diopiError_t diopiGetTensorDataConst(diopiConstTensorHandle_t tensor, const void** data);
diopiError_t diopiGetTensorShape(diopiConstTensorHandle_t tensor, diopiSize_t* shape);
diopiError_t diopiGetTensorStride(diopiConstTensorHandle_t tensor, diopiSize_t* strideInElements);
diopiError_t diopiGetTensorDtype(diopiConstTensorHandle_t tensor, diopiDtype_t* dtype);
diopiError_t diopiGetTensorNumel(diopiConstTensorHandle_t tensor, int64_t* count);
/* Optional on the caller's side (weak): test the address before calling. */
DIOPI_ATTR_WEAK diopiError_t diopiGetTensorDevice(diopiConstTensorHandle_t tensor, diopiDevice_t* where);
DIOPI_ATTR_WEAK diopiError_t diopiGetTensorElemSize(diopiConstTensorHandle_t tensor, int64_t* bytesPerElement);
DIOPI_ATTR_WEAK diopiError_t diopiGetTensorStoragePtr(diopiConstTensorHandle_t tensor, void** storage);
DIOPI_ATTR_WEAK diopiError_t diopiGetTensorStorageOffset(diopiConstTensorHandle_t tensor, int64_t* offset);
DIOPI_ATTR_WEAK diopiError_t diopiGetTensorStorageNbytes(diopiConstTensorHandle_t tensor, size_t* bytes);
DIOPI_ATTR_WEAK diopiError_t diopiGetTensorDeviceIndex(diopiConstTensorHandle_t tensor, diopiDeviceIndex_t* index);
DIOPI_ATTR_WEAK diopiError_t diopiGetCurrentDeviceIndex(diopiDeviceIndex_t* index);

/* ---- stream and scratch memory, implemented by the caller (reference: diopirt.h:145-150) ----
 * Whatever diopiRequireTensor / diopiRequireBuffer hand out belongs to the
 * context: the library never frees it and never keeps the pointer past the
 * call that asked for it.  A null stride asks for a dense tensor. */
diopiError_t diopiGetStream(diopiContextHandle_t ctx, diopiStreamHandle_t* nativeStream);
diopiError_t diopiRequireTensor(diopiContextHandle_t ctx, diopiTensorHandle_t* made, const diopiSize_t* shape, const diopiSize_t* strideOrNull,
                                const diopiDtype_t dtype, const diopiDevice_t where);
DIOPI_ATTR_WEAK diopiError_t diopiRequireBuffer(diopiContextHandle_t ctx, diopiTensorHandle_t* made, int64_t bytes, diopiDevice_t where);

/* ---- profiler scopes, optional (reference: diopirt.h:161-162) ---- */
DIOPI_ATTR_WEAK diopiError_t diopiRecordStart(const char* scopeName, void** scope);
DIOPI_ATTR_WEAK diopiError_t diopiRecordEnd(void** scope);

#if defined(__cplusplus)
}
#endif

#endif /* DIOPI_ROCM_INCLUDE_DIOPI_DIOPIRT_H_ */
