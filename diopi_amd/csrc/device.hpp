// Device-side building blocks for the gfx950 kernels: element types and their
// fp32 conversions, 128-bit global accesses, wavefront (64-lane) reductions.
#ifndef DIOPI_ROCM_CSRC_DEVICE_HPP_
#define DIOPI_ROCM_CSRC_DEVICE_HPP_

#include <hip/hip_runtime.h>

#include <cstdint>

namespace rocm {

constexpr int kWave = 64;  // CDNA wavefront width
constexpr int kNumXcd = 8;  // accelerator dies of an MI355X: consecutive work-groups of a launch go to them round-robin

using half_t = _Float16;
using bf16_t = __bf16;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// The arithmetic type a given element type accumulates in (fp32, or fp64 for fp64 data),
// matching at::acc_type as used by the reference (layer_norm_cuda_kernel.cu:971).
template <typename T>
struct AccType {
    using type = float;
};
template <>
struct AccType<double> {
    using type = double;
};

template <typename T>
__device__ __forceinline__ float toFloat(T v) {
    return static_cast<float>(v);
}

// Round-to-nearest-even conversion from fp32 to the element type.
template <typename T>
__device__ __forceinline__ T fromFloat(float v) {
    return static_cast<T>(v);
}

// fp64 sums are narrowed through the accumulation type of the destination.
template <typename T>
__device__ __forceinline__ T fromDouble(double v) {
    if constexpr (sizeof(T) == 8) {
        return v;
    } else {
        return static_cast<T>(static_cast<float>(v));
    }
}

// A 16-byte packet of elements, the unit of every vectorised global access.
template <typename T>
struct Pack16 {
    static constexpr int N = 16 / sizeof(T);
    union {
        u32x4 raw;
        T e[N];
    };
    __device__ __forceinline__ Pack16() {}
};

template <typename T>
__device__ __forceinline__ Pack16<T> loadPack(const T* p) {
    Pack16<T> v;
    v.raw = *reinterpret_cast<const u32x4*>(p);
    return v;
}

// Streaming variants: data that is touched once should not displace reusable lines.
template <typename T>
__device__ __forceinline__ Pack16<T> loadPackStream(const T* p) {
    Pack16<T> v;
    v.raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return v;
}

template <typename T>
__device__ __forceinline__ void storePack(T* p, const Pack16<T>& v) {
    *reinterpret_cast<u32x4*>(p) = v.raw;
}

template <typename T>
__device__ __forceinline__ void storePackStream(T* p, const Pack16<T>& v) {
    __builtin_nontemporal_store(v.raw, reinterpret_cast<u32x4*>(p));
}

// Butterfly reductions over the 64 lanes of a wavefront; every lane ends with the result.
template <typename T>
__device__ __forceinline__ T waveSum(T v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

template <typename T>
__device__ __forceinline__ T waveMax(T v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        T o = __shfl_xor(v, off, kWave);
        v = o > v ? o : v;
    }
    return v;
}

// v_mfma_f32_16x16x32 on 16-bit operands: lane l supplies row/column l % 16 and the 8 consecutive k
// values 8 * (l / 16) .. +7 of A and of B; it receives rows 4 * (l / 16) .. +3 of column l % 16 of C.
template <typename T>
struct Mfma16;
template <>
struct Mfma16<half_t> {
    using Frag = f16x8;
    static __device__ __forceinline__ f32x4 mma(Frag a, Frag b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};
template <>
struct Mfma16<bf16_t> {
    using Frag = bf16x8;
    static __device__ __forceinline__ f32x4 mma(Frag a, Frag b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};

// Reductions over the 16 lanes of a DPP row (quad permutes, then half-row and full-row mirrors); every lane of the
// row ends with the result.  Four VALU moves instead of four trips through the LDS crossbar.
template <int CTRL>
__device__ __forceinline__ float dppMove(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float rowMax16(float v) {
    v = fmaxf(v, dppMove<0xB1>(v));   // quad_perm [1,0,3,2]
    v = fmaxf(v, dppMove<0x4E>(v));   // quad_perm [2,3,0,1]
    v = fmaxf(v, dppMove<0x141>(v));  // row_half_mirror
    v = fmaxf(v, dppMove<0x140>(v));  // row_mirror
    return v;
}
__device__ __forceinline__ float rowSum16(float v) {
    v += dppMove<0xB1>(v);
    v += dppMove<0x4E>(v);
    v += dppMove<0x141>(v);
    v += dppMove<0x140>(v);
    return v;
}

// Reads an index tensor element as int64 whatever its storage width.
__device__ __forceinline__ int64_t loadIndex(const void* base, int64_t i, bool is64) {
    return is64 ? reinterpret_cast<const int64_t*>(base)[i] : static_cast<int64_t>(reinterpret_cast<const int32_t*>(base)[i]);
}

// Longest first.  Work-groups start in the order of their index and a compute unit holds a few at a time, so when their
// work is ragged the order decides how long the last ones run alone.  Called by all 64 lanes of one wave: returns which
// of n <= 256 items (4 per lane) has the r-th largest size, ties by item number, by bisection on the size (sizeOf(j) in
// [0, maxSize]): log2(maxSize) rounds of 4 compares and 4 ballots, a few hundred instructions that the streaming of the
// other resident work-groups hides.  Every r in [0, n) gets a different item.
constexpr int kRankedItems = 4 * kWave;
template <typename SizeOf>
__device__ __forceinline__ int itemOfRank(int r, int n, int maxSize, SizeOf sizeOf) {
    const int l = threadIdx.x % kWave;
    int sz[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int j = l + kWave * k;
        sz[k] = j < n ? sizeOf(j) : -1;  // no such item: behind every real one
    }
    auto atLeast = [&](int64_t v) {  // items of at least this size
        int c = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) c += __builtin_popcountll(__ballot(static_cast<int64_t>(sz[k]) >= v));
        return c;
    };
    int64_t lo = 0, hi = static_cast<int64_t>(maxSize) + 1;  // atLeast(lo) > r >= atLeast(hi); 64 bits: maxSize may be INT32_MAX
    while (hi - lo > 1) {
        const int64_t mid = lo + (hi - lo) / 2;
        if (atLeast(mid) > r) {
            lo = mid;
        } else {
            hi = mid;
        }
    }
    int t = r - atLeast(lo + 1);  // position among the items of exactly this size
    int found = r;
    bool done = false;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const unsigned long long eq = __ballot(static_cast<int64_t>(sz[k]) == lo);
        const int before = __builtin_popcountll(eq & ((1ull << l) - 1ull));
        const unsigned long long hit = __ballot(static_cast<int64_t>(sz[k]) == lo && before == t);
        if (!done && hit != 0ull) {
            found = __builtin_ctzll(hit) + kWave * k;
            done = true;
        }
        t -= __builtin_popcountll(eq);
    }
    return found;
}

// The same without a branch: two loads whatever the width (for 32-bit storage the second one re-reads the element),
// combined afterwards.  A load inside a branch makes the compiler wait for it before the branch ends; this form lets
// the value stay in flight until its first use.
__device__ __forceinline__ int64_t loadIndexInFlight(const void* base, int64_t i, bool is64) {
    const char* p = reinterpret_cast<const char*>(base) + i * (is64 ? 8 : 4);
    const uint32_t lo = *reinterpret_cast<const uint32_t*>(p);
    const uint32_t hi = *reinterpret_cast<const uint32_t*>(p + (is64 ? 4 : 0));
    return is64 ? static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo) : static_cast<int64_t>(static_cast<int32_t>(lo));
}

// A pointer every lane of the wave holds the same value of, moved to scalar registers (buffer descriptors live there).
template <typename T>
__device__ __forceinline__ T* uniformPointer(T* p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
    return reinterpret_cast<T*>((static_cast<uint64_t>(hi) << 32) | lo);
}

// Raw buffer descriptor over `bytes` bytes at `base`: loads past the end return zero and stores past it are dropped by
// the hardware, so a guarded access needs no branch.
constexpr int kRawBufferWord3 = 0x00020000;
__device__ __forceinline__ __amdgpu_buffer_rsrc_t rawBuffer(const void* base, int bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, kRawBufferWord3);
}

}  // namespace rocm

#endif  // DIOPI_ROCM_CSRC_DEVICE_HPP_
