// Error buffer, handle unwrapping and context services for the gfx950 DIOPI operators.
#include "common.hpp"
#include "decode.hpp"

#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <utility>

namespace rocm {

// ---- last error ------------------------------------------------------------
// The text returned by diopiGetLastErrorString() is "<device error>; other error: <message>", as in
// impl/torch/functions/error.cpp:13-29 of the reference.  The reference keeps one process-wide buffer behind a
// mutex, which still hands the caller a pointer another thread may be rewriting; here every host thread has its
// own message, so the pointer stays valid and describes the calling thread's last failure.
namespace {
thread_local char gLastErrorText[4096] = {0};
thread_local char gLastErrorOther[2048] = {0};
thread_local char gLastHipError[256] = "no error";
}  // namespace

void setLastError(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(gLastErrorOther, sizeof(gLastErrorOther), fmt, ap);
    va_end(ap);
}

void setLastErrorAt(const char* file, int line, const char* fmt, ...) {
    const char* base = std::strrchr(file, '/');
    int n = snprintf(gLastErrorOther, sizeof(gLastErrorOther), "%s:%d: ", base ? base + 1 : file, line);
    if (n < 0 || n >= static_cast<int>(sizeof(gLastErrorOther))) return;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(gLastErrorOther + n, sizeof(gLastErrorOther) - n, fmt, ap);
    va_end(ap);
}

void noteHipError(hipError_t err) {
    snprintf(gLastHipError, sizeof(gLastHipError), "%s", hipGetErrorString(err));
}

static const char* lastErrorString() {
    snprintf(gLastErrorText, sizeof(gLastErrorText), "hip error: %s; other error: %s", gLastHipError, gLastErrorOther);
    return gLastErrorText;
}

// ---- dtype helpers ------------------------------------------------------------
int64_t itemsizeOf(diopiDtype_t dtype) {
    switch (dtype) {
        case diopi_dtype_int8:
        case diopi_dtype_uint8:
        case diopi_dtype_bool:
            return 1;
        case diopi_dtype_int16:
        case diopi_dtype_uint16:
        case diopi_dtype_float16:
        case diopi_dtype_bfloat16:
            return 2;
        case diopi_dtype_int32:
        case diopi_dtype_uint32:
        case diopi_dtype_float32:
        case diopi_dtype_tfloat32:
            return 4;
        case diopi_dtype_int64:
        case diopi_dtype_uint64:
        case diopi_dtype_float64:
            return 8;
        default:
            return 0;
    }
}

const char* dtypeName(diopiDtype_t dtype) {
    switch (dtype) {
        case diopi_dtype_int8: return "int8";
        case diopi_dtype_uint8: return "uint8";
        case diopi_dtype_int16: return "int16";
        case diopi_dtype_uint16: return "uint16";
        case diopi_dtype_int32: return "int32";
        case diopi_dtype_uint32: return "uint32";
        case diopi_dtype_int64: return "int64";
        case diopi_dtype_uint64: return "uint64";
        case diopi_dtype_float16: return "float16";
        case diopi_dtype_float32: return "float32";
        case diopi_dtype_float64: return "float64";
        case diopi_dtype_bool: return "bool";
        case diopi_dtype_bfloat16: return "bfloat16";
        default: return "unsupported";
    }
}

int64_t TensorView::itemsize() const { return itemsizeOf(dtype); }

bool TensorView::isContiguous() const {
    if (numel == 0) return true;  // nothing to address
    int64_t expect = 1;
    for (int i = ndim - 1; i >= 0; --i) {
        if (shape[i] == 1) continue;  // stride of a unit dimension is irrelevant
        if (stride[i] != expect) return false;
        expect *= shape[i];
    }
    return true;
}

bool TensorView::sameShape(const TensorView& o) const {
    if (ndim != o.ndim) return false;
    for (int i = 0; i < ndim; ++i) {
        if (shape[i] != o.shape[i]) return false;
    }
    return true;
}

diopiError_t unwrap(diopiConstTensorHandle_t th, const char* name, TensorView* view) {
    ROCM_CHECK(th != nullptr, "tensor '%s' is a null handle", name);
    diopiSize_t shape{nullptr, 0}, stride{nullptr, 0};
    ROCM_CHECK(diopiGetTensorShape(th, &shape) == diopiSuccess, "diopiGetTensorShape failed for '%s'", name);
    ROCM_CHECK(diopiGetTensorStride(th, &stride) == diopiSuccess, "diopiGetTensorStride failed for '%s'", name);
    ROCM_CHECK(shape.len >= 0 && shape.len <= kMaxDims, "tensor '%s' has rank %lld; at most %d dimensions are supported", name,
               static_cast<long long>(shape.len), kMaxDims);
    ROCM_CHECK(stride.len == shape.len, "tensor '%s': stride rank %lld differs from shape rank %lld", name, static_cast<long long>(stride.len),
               static_cast<long long>(shape.len));
    view->ndim = static_cast<int>(shape.len);
    view->numel = 1;
    for (int i = 0; i < view->ndim; ++i) {
        view->shape[i] = shape.data[i];
        view->stride[i] = stride.data[i];
        ROCM_CHECK(shape.data[i] >= 0, "tensor '%s' has a negative extent", name);
        view->numel *= shape.data[i];
    }
    ROCM_CHECK(diopiGetTensorDtype(th, &view->dtype) == diopiSuccess, "diopiGetTensorDtype failed for '%s'", name);
    view->device = diopi_device;
    if (diopiGetTensorDevice != nullptr) {
        ROCM_CHECK(diopiGetTensorDevice(th, &view->device) == diopiSuccess, "diopiGetTensorDevice failed for '%s'", name);
    }
    const void* p = nullptr;
    ROCM_CHECK(diopiGetTensorDataConst(th, &p) == diopiSuccess, "diopiGetTensorDataConst failed for '%s'", name);
    view->data = const_cast<void*>(p);
    ROCM_CHECK(view->numel == 0 || view->data != nullptr, "tensor '%s' has no data pointer", name);
    return diopiSuccess;
}

diopiError_t requireDeviceContiguous(const TensorView& v, const char* name) {
    ROCM_CHECK(v.device == diopi_device, "tensor '%s' must live in device memory", name);
    ROCM_CHECK(v.isContiguous(), "tensor '%s' must be contiguous", name);
    return diopiSuccess;
}

// ---- context services ------------------------------------------------------------
diopiError_t getStream(diopiContextHandle_t ctx, hipStream_t* stream) {
    ROCM_CHECK(ctx != nullptr, "the context handle is null");
    diopiStreamHandle_t handle = nullptr;
    ROCM_CHECK(diopiGetStream(ctx, &handle) == diopiSuccess, "diopiGetStream failed");
    *stream = static_cast<hipStream_t>(handle);
    return diopiSuccess;
}

diopiError_t requireScratch(diopiContextHandle_t ctx, int64_t bytes, void** ptr) {
    ROCM_CHECK(ctx != nullptr, "the context handle is null");
    diopiTensorHandle_t t = nullptr;
    if (diopiRequireBuffer != nullptr) {
        ROCM_CHECK(diopiRequireBuffer(ctx, &t, bytes, diopi_device) == diopiSuccess && t != nullptr, "diopiRequireBuffer(%lld bytes) failed",
                   static_cast<long long>(bytes));
    } else {
        diopiSize_t size{&bytes, 1};
        ROCM_CHECK(diopiRequireTensor(ctx, &t, &size, nullptr, diopi_dtype_int8, diopi_device) == diopiSuccess && t != nullptr,
                   "diopiRequireTensor(%lld bytes) failed", static_cast<long long>(bytes));
    }
    ROCM_CHECK(diopiGetTensorData(t, ptr) == diopiSuccess && *ptr != nullptr, "scratch tensor has no data pointer");
    return diopiSuccess;
}

namespace {
__global__ void zeroFillKernel(unsigned char* p, int64_t bytes) {
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < bytes; i += static_cast<int64_t>(gridDim.x) * blockDim.x) p[i] = 0;
}
}  // namespace

diopiError_t zeroFill(hipStream_t stream, void* ptr, int64_t bytes) {
    if (bytes <= 0) return diopiSuccess;
    int64_t blocks = ceilDiv(bytes, 256);
    if (blocks > 1024) blocks = 1024;
    hipLaunchKernelGGL(zeroFillKernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, static_cast<unsigned char*>(ptr), bytes);
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
}

diopiError_t prepareDecode(const TensorView& logits, const TensorView& qOrOut, const TensorView& cache, const TensorView& bLoc, const TensorView& bStartLoc,
                           const TensorView& bSeqLen, int maxInputLen, DecodeArgs* a, bool* empty) {
    *empty = false;
    ROCM_CALL(requireDeviceContiguous(logits, "logits"));
    ROCM_CALL(requireDeviceContiguous(qOrOut, "q/out"));
    ROCM_CALL(requireDeviceContiguous(cache, "k/v cache"));
    ROCM_CALL(requireDeviceContiguous(bLoc, "b_loc"));
    ROCM_CALL(requireDeviceContiguous(bStartLoc, "b_start_loc"));
    ROCM_CALL(requireDeviceContiguous(bSeqLen, "b_seq_len"));
    ROCM_CHECK(qOrOut.ndim == 3 && cache.ndim == 3 && logits.ndim == 2 && bLoc.ndim == 2,
               "expected q/out [B,H,D], cache [slots,Hkv,D], logits [H,cols], b_loc [B,N]");
    ROCM_CHECK(bStartLoc.ndim == 1 && bSeqLen.ndim == 1, "b_start_loc and b_seq_len must be one-dimensional");
    ROCM_CHECK(isFloatDtype(qOrOut.dtype) && cache.dtype == qOrOut.dtype && logits.dtype == qOrOut.dtype,
               "q/out, the cache and the logits must share one floating dtype (got %s, %s, %s)", dtypeName(qOrOut.dtype), dtypeName(cache.dtype),
               dtypeName(logits.dtype));
    ROCM_CHECK(isIndexDtype(bLoc.dtype) && isIndexDtype(bStartLoc.dtype) && isIndexDtype(bSeqLen.dtype),
               "b_loc, b_start_loc and b_seq_len must be int32 or int64");
    const int64_t B = bLoc.shape[0];
    ROCM_CHECK(qOrOut.shape[0] == B && bStartLoc.shape[0] == B && bSeqLen.shape[0] == B,
               "q/out, b_start_loc and b_seq_len must have b_loc's batch size %lld", static_cast<long long>(B));
    const int64_t H = qOrOut.shape[1], D = qOrOut.shape[2], Hkv = cache.shape[1];
    ROCM_CHECK(cache.shape[2] == D, "head size mismatch between q/out (%lld) and the cache (%lld)", static_cast<long long>(D),
               static_cast<long long>(cache.shape[2]));
    ROCM_CHECK(Hkv > 0 && H % Hkv == 0, "query heads (%lld) must be a multiple of kv heads (%lld)", static_cast<long long>(H),
               static_cast<long long>(Hkv));
    ROCM_CHECK(logits.shape[0] == H, "the logits tensor must have %lld rows (one per query head), got %lld", static_cast<long long>(H),
               static_cast<long long>(logits.shape[0]));
    ROCM_CHECK(maxInputLen >= 0 && maxInputLen <= bLoc.shape[1], "max_input_len %d exceeds the width of b_loc (%lld)", maxInputLen,
               static_cast<long long>(bLoc.shape[1]));
    ROCM_CHECK(B <= 65535, "batch size %lld exceeds the launch limit of 65535", static_cast<long long>(B));
    ROCM_CHECK(H <= 65535 && D <= 65535, "head count %lld / head size %lld out of range", static_cast<long long>(H), static_cast<long long>(D));
    if (B == 0 || maxInputLen == 0 || H == 0 || D == 0 || logits.numel == 0) {
        *empty = true;
        return diopiSuccess;
    }
    ROCM_CHECK(cache.shape[0] > 0, "the kv cache has no rows");
    a->bLoc = bLoc.data;
    a->bStartLoc = bStartLoc.data;
    a->bSeqLen = bSeqLen.data;
    a->bLocStride = bLoc.shape[1];
    a->numSlots = cache.shape[0];
    a->logitCols = logits.shape[1];
    a->batch = static_cast<int>(B);
    a->H = static_cast<int>(H);
    a->Hkv = static_cast<int>(Hkv);
    a->G = static_cast<int>(H / Hkv);
    a->D = static_cast<int>(D);
    a->maxInputLen = maxInputLen;
    a->loc64 = bLoc.dtype == diopi_dtype_int64;
    a->start64 = bStartLoc.dtype == diopi_dtype_int64;
    a->len64 = bSeqLen.dtype == diopi_dtype_int64;
    return diopiSuccess;
}

const DeviceInfo& deviceInfo() {
    static const DeviceInfo info = [] {
        DeviceInfo d;
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) {
            d.numCU = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : d.numCU;
            d.maxSharedPerBlock = static_cast<int>(prop.sharedMemPerBlock);
            int optin = 0;
            if (hipDeviceGetAttribute(&optin, hipDeviceAttributeSharedMemPerBlockOptin, dev) == hipSuccess && optin > 0) {
                d.maxSharedOptin = optin;
            } else {
                (void)hipGetLastError();
                d.maxSharedOptin = d.maxSharedPerBlock;
            }
        } else {
            (void)hipGetLastError();
        }
        return d;
    }();
    return info;
}

diopiError_t grantDynamicLds(const void* kernel, int bytes) {
    static std::mutex mtx;
    static std::map<std::pair<const void*, int>, int> granted;  // (kernel, device) -> bytes granted so far
    int dev = 0;
    ROCM_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(mtx);
    int& have = granted[std::make_pair(kernel, dev)];
    if (have >= bytes) return diopiSuccess;
    ROCM_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    have = bytes;
    return diopiSuccess;
}

}  // namespace rocm

// ---- library identification (reference: impl/torch/functions/functions.cpp:37-66) ----
extern "C" {

const char* diopiGetVendorName() { return "RocmDevice"; }

const char* diopiGetImplVersion() {
    static char version[256] = {0};
    static std::once_flag once;
    std::call_once(once, [] {
        snprintf(version, sizeof(version), "HIP Version: %d; DIOPI Version: %d.%d.%d; arch gfx950", HIP_VERSION, DIOPI_VER_MAJOR, DIOPI_VER_MINOR,
                 DIOPI_VER_PATCH);
    });
    return version;
}

const char* diopiGetLastErrorString() { return rocm::lastErrorString(); }

}  // extern "C"
