/*
 * DIOPI runtime interface, restated for the gfx950 operator library.
 *
 * This header carries the part of the DIOPI C ABI that the operator library
 * and its caller share: value types, opaque handles and the callbacks the
 * library imports from whoever owns the tensors.  Every declaration below is
 * binary- and source-compatible with the reference header it restates
 * (reference: proto/include/diopi/diopirt.h, line numbers cited per block), so
 * a translation unit may be compiled against either header directory.
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

/* reference: diopirt.h:22-25 */
#define DIOPI_VER_MAJOR 1
#define DIOPI_VER_MINOR 0
#define DIOPI_VER_PATCH 0
#define DIOPI_VERSION (DIOPI_VER_MAJOR * 1000 + DIOPI_VER_MINOR * 100 + DIOPI_VER_PATCH)

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

/* reference: diopirt.h:81-87 */
typedef struct {
    diopiDtype_t stype;
    union {
        double fval;
        int64_t ival;
    };
} diopiScalar_t;

/* reference: diopirt.h:89-93 (unused by the LLaMA inference operators, kept for layout parity) */
typedef enum { Contiguous = 0, ChannelsLast = 1, ChannelsLast3d = 2, Preserve = 3, ChannelsLast1d = 4 } diopiMemoryFormat_t;
typedef enum { ReductionNone, ReductionMean, ReductionSum, ReductionEND } diopiReduction_t;
typedef enum { RoundModeNone, RoundModeTrunc, RoundModeFloor, RoundModeEND } diopiRoundMode_t;

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

/* reference: diopirt.h:117 */
extern DIOPI_API const char* diopiGetVersion();

/* ---- tensor accessors, implemented by the caller (reference: diopirt.h:122-140) ----
 * diopiGetTensorData already includes any storage offset. Shape/Stride return
 * pointers into caller-owned memory that lives as long as the tensor. */
extern DIOPI_RT_API diopiError_t diopiGetTensorData(diopiTensorHandle_t th, void**);
extern DIOPI_RT_API diopiError_t diopiGetTensorDataConst(diopiConstTensorHandle_t th, const void**);
extern DIOPI_RT_API diopiError_t diopiGetTensorShape(diopiConstTensorHandle_t th, diopiSize_t* size);
extern DIOPI_RT_API diopiError_t diopiGetTensorStride(diopiConstTensorHandle_t th, diopiSize_t* stride);
extern DIOPI_RT_API diopiError_t diopiGetTensorDtype(diopiConstTensorHandle_t th, diopiDtype_t* dtype);
extern DIOPI_RT_API diopiError_t diopiGetTensorNumel(diopiConstTensorHandle_t th, int64_t* numel);
/* the following accessors are optional on the caller's side: test for null before use */
extern DIOPI_RT_API DIOPI_ATTR_WEAK diopiError_t diopiGetTensorDevice(diopiConstTensorHandle_t th, diopiDevice_t* device);
extern DIOPI_RT_API DIOPI_ATTR_WEAK diopiError_t diopiGetTensorElemSize(diopiConstTensorHandle_t th, int64_t* itemsize);
extern DIOPI_RT_API DIOPI_ATTR_WEAK diopiError_t diopiGetTensorStoragePtr(diopiConstTensorHandle_t th, void** pStoragePtr);
extern DIOPI_RT_API DIOPI_ATTR_WEAK diopiError_t diopiGetTensorStorageOffset(diopiConstTensorHandle_t th, int64_t* pOffset);
extern DIOPI_RT_API DIOPI_ATTR_WEAK diopiError_t diopiGetTensorStorageNbytes(diopiConstTensorHandle_t th, size_t* pNbytes);
extern DIOPI_RT_API DIOPI_ATTR_WEAK diopiError_t diopiGetTensorDeviceIndex(diopiConstTensorHandle_t th, diopiDeviceIndex_t* pDevIndex);
extern DIOPI_RT_API DIOPI_ATTR_WEAK diopiError_t diopiGetCurrentDeviceIndex(diopiDeviceIndex_t* pDevIndex);

/* ---- stream and scratch memory, implemented by the caller (reference: diopirt.h:145-150) ----
 * Everything obtained through diopiRequireTensor/diopiRequireBuffer belongs to
 * the context: the library never frees it and never keeps the pointer past
 * the call that asked for it. */
extern DIOPI_RT_API diopiError_t diopiGetStream(diopiContextHandle_t ctx, diopiStreamHandle_t* stream);
extern DIOPI_RT_API diopiError_t diopiRequireTensor(diopiContextHandle_t ctx, diopiTensorHandle_t* tensor, const diopiSize_t* size, const diopiSize_t* stride,
                                                    const diopiDtype_t dtype, const diopiDevice_t device);
extern DIOPI_RT_API DIOPI_ATTR_WEAK diopiError_t diopiRequireBuffer(diopiContextHandle_t ctx, diopiTensorHandle_t* tensor, int64_t num_bytes,
                                                                    diopiDevice_t device);

/* ---- profiler scopes, optional (reference: diopirt.h:161-162) ---- */
extern DIOPI_RT_API DIOPI_ATTR_WEAK diopiError_t diopiRecordStart(const char* record_name, void** record);
extern DIOPI_RT_API DIOPI_ATTR_WEAK diopiError_t diopiRecordEnd(void** record);

#if defined(__cplusplus)
}
#endif

#endif /* DIOPI_ROCM_INCLUDE_DIOPI_DIOPIRT_H_ */
