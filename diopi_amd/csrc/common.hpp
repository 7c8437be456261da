// Host-side glue shared by the operator entry points: handle unwrapping through
// the diopirt callbacks, argument validation, error reporting, scratch and
// stream access.  Plays the role of impl/cuda/helper.hpp:55-135 and
// impl/torch/helper.hpp:39-75 of the reference, without any tensor framework.
#ifndef DIOPI_ROCM_CSRC_COMMON_HPP_
#define DIOPI_ROCM_CSRC_COMMON_HPP_

#include <diopi/diopirt.h>
#include <diopi/functions.h>
#include <diopi/functions_ext.h>
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <exception>

namespace rocm {

// ---- last-error buffer (error.cpp) -----------------------------------------
void setLastError(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
void noteHipError(hipError_t err);

// Fail the current entry point: record "<file>:<line>: <message>" and return diopiErrorOccurred.
#define ROCM_CHECK(cond, ...)                                                       \
    do {                                                                            \
        if (!(cond)) {                                                              \
            ::rocm::setLastErrorAt(__FILE__, __LINE__, __VA_ARGS__);                \
            return diopiErrorOccurred;                                              \
        }                                                                           \
    } while (0)

#define ROCM_CALL(expr)                          \
    do {                                         \
        diopiError_t rocmCallRet_ = (expr);      \
        if (rocmCallRet_ != diopiSuccess) {      \
            return rocmCallRet_;                 \
        }                                        \
    } while (0)

#define ROCM_HIP(expr)                                                                                   \
    do {                                                                                                 \
        hipError_t rocmHipRet_ = (expr);                                                                 \
        if (rocmHipRet_ != hipSuccess) {                                                                 \
            ::rocm::noteHipError(rocmHipRet_);                                                           \
            ::rocm::setLastErrorAt(__FILE__, __LINE__, "%s failed: %s", #expr, hipGetErrorString(rocmHipRet_)); \
            return diopiErrorOccurred;                                                                   \
        }                                                                                                \
    } while (0)

// Checked right after every kernel launch; launch-configuration errors surface here.
#define ROCM_LAUNCH_CHECK() ROCM_HIP(hipGetLastError())

void setLastErrorAt(const char* file, int line, const char* fmt, ...) __attribute__((format(printf, 3, 4)));

// No C++ exception may cross the C ABI: every extern "C" body is wrapped in these.
#define ROCM_ENTRY_BEGIN try {
#define ROCM_ENTRY_END                                                   \
    }                                                                    \
    catch (const std::exception& e) {                                    \
        ::rocm::setLastError("unhandled exception: %s", e.what());       \
        return diopiErrorOccurred;                                       \
    }                                                                    \
    catch (...) {                                                        \
        ::rocm::setLastError("unhandled non-standard exception");        \
        return diopiErrorOccurred;                                       \
    }

// ---- tensor view -------------------------------------------------------------
constexpr int kMaxDims = 8;

struct TensorView {
    void* data = nullptr;
    diopiDtype_t dtype = diopi_dtype_unsupported;
    diopiDevice_t device = diopi_device;
    int ndim = 0;
    int64_t shape[kMaxDims] = {0};
    int64_t stride[kMaxDims] = {0};
    int64_t numel = 0;

    int64_t size(int i) const { return shape[i < 0 ? i + ndim : i]; }
    int64_t itemsize() const;
    int64_t nbytes() const { return numel * itemsize(); }
    bool isContiguous() const;
    bool sameShape(const TensorView& o) const;
};

int64_t itemsizeOf(diopiDtype_t dtype);
const char* dtypeName(diopiDtype_t dtype);

// Fills `view` from the handle; fails on null handles, rank > kMaxDims or callback errors.
diopiError_t unwrap(diopiConstTensorHandle_t th, const char* name, TensorView* view);

// Common precondition of every operator: device memory and dense row-major layout.
diopiError_t requireDeviceContiguous(const TensorView& v, const char* name);

inline bool isFloatDtype(diopiDtype_t d) {
    return d == diopi_dtype_float16 || d == diopi_dtype_bfloat16 || d == diopi_dtype_float32 || d == diopi_dtype_float64;
}
inline bool isIndexDtype(diopiDtype_t d) { return d == diopi_dtype_int32 || d == diopi_dtype_int64; }

// ---- context services ----------------------------------------------------------
diopiError_t getStream(diopiContextHandle_t ctx, hipStream_t* stream);
// Device scratch owned by the context (diopiRequireBuffer, or diopiRequireTensor(int8) when the
// caller does not provide the optional callback).
diopiError_t requireScratch(diopiContextHandle_t ctx, int64_t bytes, void** ptr);

// Clears `bytes` bytes of device memory with a kernel (safe to record into a HIP graph).
diopiError_t zeroFill(hipStream_t stream, void* ptr, int64_t bytes);

// Properties of the current device, queried once per process.
struct DeviceInfo {
    int numCU = 256;
    int maxSharedPerBlock = 65536;
    int maxSharedOptin = 65536;  // LDS a work-group may use with dynamic shared memory granted explicitly
};
const DeviceInfo& deviceInfo();

// Lets `kernel` use `bytes` of dynamic LDS beyond the 64 KiB default, once per kernel and device (the attribute belongs
// to the device the call runs on; a process may hold several).
diopiError_t grantDynamicLds(const void* kernel, int bytes);

inline int64_t ceilDiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace rocm

#endif  // DIOPI_ROCM_CSRC_COMMON_HPP_
