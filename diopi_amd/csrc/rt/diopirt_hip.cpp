// HIP-backed caller side of the DIOPI runtime interface (see include/diopirt_hip.h).
//
// Mirrors what diopi_test/diopi_stub/csrc/litert.cpp:209-330 of the reference
// provides to an operator library: tensor accessors, the context's stream and
// context-owned scratch tensors.  Scratch comes from a per-context pool so that
// repeated operator calls do not hit hipMalloc/hipFree.
#include <conform_test.h>
#include <diopirt_hip.h>
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

extern "C" int64_t diopirtItemsize(diopiDtype_t dtype) {
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
        case diopi_dtype_complex32:
            return 4;
        case diopi_dtype_int64:
        case diopi_dtype_uint64:
        case diopi_dtype_float64:
        case diopi_dtype_complex64:
            return 8;
        case diopi_dtype_complex128:
            return 16;
        default:
            return 0;
    }
}

// The handle types are opaque to the operator library; only this file sees inside.
struct diopiTensor {
    std::vector<int64_t> shape;
    std::vector<int64_t> stride;
    diopiDtype_t dtype = diopi_dtype_unsupported;
    diopiDevice_t device = diopi_device;
    int64_t numel = 0;
    void* data = nullptr;
    int64_t capacity = 0;  // bytes of the pool block behind `data`; 0 for wrapped memory
};

struct diopiContext {
    hipStream_t stream = nullptr;
    bool ownsStream = false;
    bool adopted = false;
    std::mutex mtx;
    std::vector<diopiTensor*> live;                     // handed out since the last clear
    std::multimap<int64_t, void*> freeDevice;           // capacity -> block
    std::multimap<int64_t, void*> freeHost;
    int64_t inUse = 0, peak = 0, mallocCount = 0;

    hipStream_t getStream() {
        std::lock_guard<std::mutex> lock(mtx);
        if (!adopted && stream == nullptr) {
            if (hipStreamCreateWithFlags(&stream, hipStreamNonBlocking) == hipSuccess) {
                ownsStream = true;
            } else {
                stream = nullptr;
            }
        }
        return stream;
    }
};

namespace {

constexpr int64_t kBlockAlign = 1024;  // the reference stub rounds every allocation to 1 KiB (litert.hpp:57-59)

int64_t roundUp(int64_t n, int64_t a) { return (n + a - 1) / a * a; }

void* poolTake(diopiContext* ctx, int64_t bytes, diopiDevice_t device, int64_t* capacity) {
    auto& freeList = device == diopi_device ? ctx->freeDevice : ctx->freeHost;
    int64_t want = roundUp(bytes > 0 ? bytes : 1, kBlockAlign);
    auto it = freeList.lower_bound(want);
    // reuse a block only if it is not wastefully larger than the request
    if (it != freeList.end() && it->first <= 2 * want + (1 << 20)) {
        void* p = it->second;
        *capacity = it->first;
        freeList.erase(it);
        return p;
    }
    void* p = nullptr;
    if (device == diopi_device) {
        if (hipMalloc(&p, want) != hipSuccess) return nullptr;
    } else {
        p = std::malloc(want);
    }
    if (p) ctx->mallocCount++;
    *capacity = want;
    return p;
}

}  // namespace

extern "C" {

int diopirtDeviceCount(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

int diopirtDeviceClockKHz(int device) {
    int khz = 0;
    if (hipDeviceGetAttribute(&khz, hipDeviceAttributeClockRate, device) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return khz;
}

int diopirtDeviceComputeUnits(int device) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

diopiContextHandle_t diopirtContextCreate(void* stream) {
    auto* ctx = new diopiContext();
    if (stream != nullptr) {
        ctx->stream = static_cast<hipStream_t>(stream);
        ctx->adopted = true;
    }
    return ctx;
}

void diopirtContextClearTensors(diopiContextHandle_t ctx) {
    if (!ctx) return;
    std::lock_guard<std::mutex> lock(ctx->mtx);
    for (diopiTensor* t : ctx->live) {
        if (t->data) {
            (t->device == diopi_device ? ctx->freeDevice : ctx->freeHost).emplace(t->capacity, t->data);
            ctx->inUse -= t->capacity;
        }
        delete t;
    }
    ctx->live.clear();
}

void diopirtContextDestroy(diopiContextHandle_t ctx) {
    if (!ctx) return;
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    diopirtContextClearTensors(ctx);
    for (auto& kv : ctx->freeDevice) (void)hipFree(kv.second);
    for (auto& kv : ctx->freeHost) std::free(kv.second);
    if (ctx->ownsStream && ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

diopiError_t diopirtContextSynchronize(diopiContextHandle_t ctx) {
    if (!ctx) return diopiErrorOccurred;
    hipStream_t s = ctx->getStream();
    return hipStreamSynchronize(s) == hipSuccess ? diopiSuccess : diopiErrorOccurred;
}

int64_t diopirtContextScratchInUse(diopiContextHandle_t ctx) { return ctx ? ctx->inUse : 0; }
int64_t diopirtContextScratchPeak(diopiContextHandle_t ctx) { return ctx ? ctx->peak : 0; }
int64_t diopirtContextMallocCount(diopiContextHandle_t ctx) { return ctx ? ctx->mallocCount : 0; }

diopiTensorHandle_t diopirtTensorWrap(void* data, const int64_t* shape, const int64_t* stride, int64_t ndim, diopiDtype_t dtype, diopiDevice_t device) {
    if (ndim < 0 || (ndim > 0 && shape == nullptr)) return nullptr;
    auto* t = new diopiTensor();
    t->shape.assign(shape, shape + ndim);
    t->stride.resize(ndim);
    int64_t running = 1;
    t->numel = 1;
    for (int64_t i = ndim - 1; i >= 0; --i) {
        t->stride[i] = stride ? stride[i] : running;
        running *= shape[i];
        t->numel *= shape[i];
    }
    t->dtype = dtype;
    t->device = device;
    t->data = data;
    return t;
}

void diopirtTensorDestroy(diopiTensorHandle_t th) { delete th; }

void* diopirtEventCreate(void) {
    hipEvent_t ev = nullptr;
    if (hipEventCreate(&ev) != hipSuccess) return nullptr;
    return ev;
}

void diopirtEventDestroy(void* ev) {
    if (ev) (void)hipEventDestroy(static_cast<hipEvent_t>(ev));
}

diopiError_t diopirtEventRecord(void* ev, diopiContextHandle_t ctx) {
    if (!ev || !ctx) return diopiErrorOccurred;
    return hipEventRecord(static_cast<hipEvent_t>(ev), ctx->getStream()) == hipSuccess ? diopiSuccess : diopiErrorOccurred;
}

float diopirtEventElapsedMs(void* start, void* stop) {
    if (!start || !stop) return -1.f;
    if (hipEventSynchronize(static_cast<hipEvent_t>(stop)) != hipSuccess) return -1.f;
    float ms = -1.f;
    if (hipEventElapsedTime(&ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)) != hipSuccess) return -1.f;
    return ms;
}

// ---------------------------------------------------------------------------
// The callbacks of diopi/diopirt.h
// ---------------------------------------------------------------------------

diopiError_t diopiGetTensorData(diopiTensorHandle_t th, void** pptr) {
    *pptr = th->data;
    return diopiSuccess;
}

diopiError_t diopiGetTensorDataConst(diopiConstTensorHandle_t th, const void** pptr) {
    *pptr = th->data;
    return diopiSuccess;
}

diopiError_t diopiGetTensorShape(diopiConstTensorHandle_t th, diopiSize_t* size) {
    size->data = th->shape.data();
    size->len = static_cast<int64_t>(th->shape.size());
    return diopiSuccess;
}

diopiError_t diopiGetTensorStride(diopiConstTensorHandle_t th, diopiSize_t* stride) {
    stride->data = th->stride.data();
    stride->len = static_cast<int64_t>(th->stride.size());
    return diopiSuccess;
}

diopiError_t diopiGetTensorDtype(diopiConstTensorHandle_t th, diopiDtype_t* dtype) {
    *dtype = th->dtype;
    return diopiSuccess;
}

diopiError_t diopiGetTensorDevice(diopiConstTensorHandle_t th, diopiDevice_t* device) {
    *device = th->device;
    return diopiSuccess;
}

diopiError_t diopiGetTensorNumel(diopiConstTensorHandle_t th, int64_t* numel) {
    *numel = th->numel;
    return diopiSuccess;
}

diopiError_t diopiGetTensorElemSize(diopiConstTensorHandle_t th, int64_t* itemsize) {
    *itemsize = diopirtItemsize(th->dtype);
    return diopiSuccess;
}

diopiError_t diopiGetTensorStoragePtr(diopiConstTensorHandle_t th, void** pStoragePtr) {
    *pStoragePtr = th->data;
    return diopiSuccess;
}

diopiError_t diopiGetTensorStorageOffset(diopiConstTensorHandle_t, int64_t* pOffset) {
    *pOffset = 0;
    return diopiSuccess;
}

diopiError_t diopiGetTensorStorageNbytes(diopiConstTensorHandle_t th, size_t* pNbytes) {
    *pNbytes = static_cast<size_t>(th->numel * diopirtItemsize(th->dtype));
    return diopiSuccess;
}

diopiError_t diopiGetTensorDeviceIndex(diopiConstTensorHandle_t, diopiDeviceIndex_t* pDevIndex) {
    *pDevIndex = 0;
    return diopiSuccess;
}

diopiError_t diopiGetCurrentDeviceIndex(diopiDeviceIndex_t* pDevIndex) {
    *pDevIndex = 0;
    return diopiSuccess;
}

diopiError_t diopiGetStream(diopiContextHandle_t ctx, diopiStreamHandle_t* stream) {
    if (!ctx) return diopiErrorOccurred;
    *stream = ctx->getStream();
    return diopiSuccess;
}

diopiError_t diopiRequireTensor(diopiContextHandle_t ctx, diopiTensorHandle_t* tensor, const diopiSize_t* size, const diopiSize_t* stride,
                                const diopiDtype_t dtype, const diopiDevice_t device) {
    if (!ctx || !tensor || !size) return diopiErrorOccurred;
    diopiTensorHandle_t t = diopirtTensorWrap(nullptr, size->data, (stride && stride->data) ? stride->data : nullptr, size->len, dtype, device);
    if (!t) return diopiErrorOccurred;
    int64_t bytes = t->numel * diopirtItemsize(dtype);
    std::lock_guard<std::mutex> lock(ctx->mtx);
    t->data = poolTake(ctx, bytes, device, &t->capacity);
    if (!t->data) {
        delete t;
        return diopiErrorOccurred;
    }
    ctx->inUse += t->capacity;
    if (ctx->inUse > ctx->peak) ctx->peak = ctx->inUse;
    ctx->live.push_back(t);
    *tensor = t;
    return diopiSuccess;
}

diopiError_t diopiRequireBuffer(diopiContextHandle_t ctx, diopiTensorHandle_t* tensor, int64_t num_bytes, diopiDevice_t device) {
    diopiSize_t size{&num_bytes, 1};
    return diopiRequireTensor(ctx, tensor, &size, nullptr, diopi_dtype_int8, device);
}

diopiError_t diopiRecordStart(const char*, void**) { return diopiSuccess; }
diopiError_t diopiRecordEnd(void**) { return diopiSuccess; }

// ---------------------------------------------------------------------------
// The device hooks of conform_test.h, through which the reference's harness reaches the device
// (CUDA versions: impl/torch/test/conform_test.cpp:27-83).
// ---------------------------------------------------------------------------

static diopiError_t hookStatus(hipError_t err, const char* what) {
    if (err == hipSuccess) return diopiSuccess;
    std::fprintf(stderr, "%s failed: %s\n", what, hipGetErrorString(err));
    (void)hipGetLastError();
    return diopiErrorOccurred;
}

void* device_malloc(uint64_t bytes) {
    void* ptr = nullptr;
    if (hookStatus(hipMalloc(&ptr, bytes > 0 ? bytes : 1), "device_malloc") != diopiSuccess) return nullptr;
    return ptr;
}

void device_free(void* ptr) {
    if (ptr != nullptr) (void)hookStatus(hipFree(ptr), "device_free");
}

diopiError_t device_make_stream(diopiStreamHandle_t* stream) {
    if (stream == nullptr) return diopiErrorOccurred;
    hipStream_t made = nullptr;
    const diopiError_t status = hookStatus(hipStreamCreate(&made), "device_make_stream");
    *stream = made;
    return status;
}

diopiError_t device_destroy_stream(diopiStreamHandle_t stream) {
    return hookStatus(hipStreamDestroy(static_cast<hipStream_t>(stream)), "device_destroy_stream");
}

diopiError_t device_synchronize_stream(diopiStreamHandle_t stream) {
    return hookStatus(hipStreamSynchronize(static_cast<hipStream_t>(stream)), "device_synchronize_stream");
}

diopiError_t device_memcpy_h2d_async(diopiStreamHandle_t stream, void* deviceDst, const void* hostSrc, uint64_t bytes) {
    if (bytes == 0) return diopiSuccess;
    return hookStatus(hipMemcpyAsync(deviceDst, hostSrc, bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream)), "device_memcpy_h2d_async");
}

diopiError_t device_memcpy_d2h_async(diopiStreamHandle_t stream, void* hostDst, const void* deviceSrc, uint64_t bytes) {
    if (bytes == 0) return diopiSuccess;
    return hookStatus(hipMemcpyAsync(hostDst, deviceSrc, bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)), "device_memcpy_d2h_async");
}

diopiError_t device_memcpy_d2d_async(diopiStreamHandle_t stream, void* deviceDst, const void* deviceSrc, uint64_t bytes) {
    if (bytes == 0) return diopiSuccess;
    return hookStatus(hipMemcpyAsync(deviceDst, deviceSrc, bytes, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)), "device_memcpy_d2d_async");
}

diopiError_t initLibrary(void) { return diopiSuccess; }
diopiError_t finalizeLibrary(void) { return diopiSuccess; }

diopiError_t buildGeneratorState(diopiContextHandle_t ctx, diopiTensorHandle_t out) {
    if (ctx == nullptr || out == nullptr) return diopiErrorOccurred;
    const int64_t stateBytes = 808;
    const diopiSize_t shape{&stateBytes, 1};
    diopiTensorHandle_t state = nullptr;
    const diopiError_t status = diopiRequireTensor(ctx, &state, &shape, nullptr, diopi_dtype_uint8, diopi_host);
    if (status != diopiSuccess) return status;
    std::memset(state->data, 0, static_cast<size_t>(stateBytes));
    *out = *state;      // `out` now views the context's block, which stays in the context's hands
    out->capacity = 0;
    return diopiSuccess;
}

}  // extern "C"
