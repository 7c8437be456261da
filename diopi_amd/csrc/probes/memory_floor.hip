// Measurement probes for gfx950, built into lib/libdiopi_probes.so and called only by `bench.py --probe`: kernels that move
// the bytes of an operator in the operator's access pattern and do no arithmetic, so that their time is the floor the memory
// system sets for that pattern, and a loop of nothing but matrix products, whose rate is what the matrix cores sustain at the
// clock the power limit leaves them.  Not part of the operator library and not exported by it.
//
// diopiProbeTokenGather follows diopiTokenAttentionInference (reference semantics functions_lightllm.cpp:53-80): a
// work-group owns a tile of `tileTokens` consecutive tokens of one sequence, looks their cache slots up in
// b_loc[i, max_input_len - L_i + t] and reads the slots' rows (all kv heads of a token are `rowBytes` contiguous bytes); it
// then writes tokens * bytesPerToken bytes, which is what the operator's logits [H, total tokens] take for the tile, cut into
// `pieces` equal runs of consecutive bytes that lie `pieceStride` bytes apart (pieces = H is the operator's own layout: one
// run per head; fewer pieces of more bytes each are what another output layout would give).  `rowSplit` work-groups share a
// tile: each reads its 1/rowSplit of every row (the operator gives a work-group some of the kv heads) and writes every
// rowSplit-th piece.  Modes: 1 reads only, 2 writes only, 3 both; + 4 makes the reads non-temporal; + 8 gives a thread two
// loads in flight instead of sixteen (more work-groups then cover for each other's waits: which of the two is faster depends
// on the pattern, so the caller tries both).
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;

struct GatherArgs {
    const char* cache;       // [slots][rowBytes]
    const int32_t* loc;      // [batch][maxInputLen]
    const int32_t* start;    // [batch] first token of the sequence in the output
    const int32_t* length;   // [batch]
    char* out;
    int64_t pieceStride;     // bytes between the pieces of a tile
    int rowBytes;            // 16 * a power of two, at most 4096
    int partBytes;           // rowBytes / rowSplit: what one work-group reads of a row
    int maxInputLen;
    int tileTokens;
    int pieces;
    int bytesPerToken;       // output bytes a token stands for (all pieces together)
    int mode;
};

// kBatch: loads a thread issues before it looks at the first of them; two such batches are in flight
template <bool NT, int kBatch>
__global__ __launch_bounds__(kThreads) void probeTokenGather(GatherArgs a) {
    // x runs over the parts of a row, y over the sequences, z over the tiles, with the sequence rotated by the tile index:
    // work-groups that start together read neighbouring parts of the same rows and tiles of many sequences, and the
    // thinly populated late tiles of the ragged batch come last
    const int i = static_cast<int>((blockIdx.y + blockIdx.z) % gridDim.y);
    const int L = a.length[i];
    const int t0 = blockIdx.z * a.tileTokens;
    if (t0 >= L) return;
    const int n = min(a.tileTokens, L - t0);
    const int tid = threadIdx.x;
    uint32_t acc = tid;
    // the tile's slots go to LDS in one coalesced load, so that no row address waits for a load of its own
    extern __shared__ int32_t slotOf[];
    if (a.mode & 1) {
        const int32_t* slots = a.loc + static_cast<int64_t>(i) * a.maxInputLen + (a.maxInputLen - L) + t0;
        for (int t = tid; t < n; t += kThreads) slotOf[t] = slots[t];
        __syncthreads();
    }
    if (a.mode & 1) {
        const int packetsPerRow = a.partBytes / 16;
        const int rowsPerStep = kThreads / packetsPerRow;  // token rows one load instruction of the work-group covers
        const int rowSel = tid / packetsPerRow;
        const int packet = tid % packetsPerRow;
        const int steps = (n + rowsPerStep - 1) / rowsPerStep;
        auto issue = [&](u32x4 (&buf)[kBatch], int s0) {
#pragma unroll
            for (int r = 0; r < kBatch; ++r) {
                int t = (s0 + r) * rowsPerStep + rowSel;
                t = t < n ? t : n - 1;  // past the tile: the last row again (a line that is already on its way)
                const u32x4* p = reinterpret_cast<const u32x4*>(a.cache + static_cast<int64_t>(slotOf[t]) * a.rowBytes + blockIdx.x * a.partBytes + packet * 16);
                buf[r] = NT ? __builtin_nontemporal_load(p) : *p;
            }
        };
        auto take = [&](const u32x4 (&buf)[kBatch]) {
#pragma unroll
            for (int r = 0; r < kBatch; ++r) acc += buf[r].x ^ buf[r].y ^ buf[r].z ^ buf[r].w;
        };
        // every trip of the loop issues both batches (rows past the tile are the last row again): with no branch around a
        // load the compiler knows how many are outstanding at each use and waits for just the oldest, instead of for all of
        // them.  The scheduling barriers keep the order written here: without them the two uses are merged ahead of the two
        // issues and one batch is in flight instead of two.
        u32x4 b0[kBatch], b1[kBatch];
        const int padded = (steps + 2 * kBatch - 1) / (2 * kBatch) * (2 * kBatch);
        issue(b0, 0);
        __builtin_amdgcn_sched_barrier(0);
        issue(b1, kBatch);
        __builtin_amdgcn_sched_barrier(0);
        for (int s = 2 * kBatch; s < padded; s += 2 * kBatch) {
            take(b0);
            __builtin_amdgcn_sched_barrier(0);
            issue(b0, s);
            __builtin_amdgcn_sched_barrier(0);
            take(b1);
            __builtin_amdgcn_sched_barrier(0);
            issue(b1, s + kBatch);
            __builtin_amdgcn_sched_barrier(0);
        }
        take(b0);
        take(b1);
    }
    if (a.mode & 2) {
        // the tile's output as 16-byte packets: piece p starts where the tile's first token lies in run p of the output
        const int perTokenPerPiece = a.bytesPerToken / a.pieces;
        const int packetsPerPiece = n * perTokenPerPiece / 16;
        const int64_t first = (static_cast<int64_t>(a.start[i] + t0) * perTokenPerPiece) & ~int64_t(15);
        const u32x4 v = {acc, acc + 1, acc + 2, acc + 3};
        const int mine = (a.pieces - static_cast<int>(blockIdx.x) + static_cast<int>(gridDim.x) - 1) / static_cast<int>(gridDim.x);  // pieces x, x + rowSplit, ...
        for (int q = tid; q < packetsPerPiece * mine; q += kThreads) {
            const int p = (q / packetsPerPiece) * gridDim.x + blockIdx.x;
            const int within = q % packetsPerPiece;
            *reinterpret_cast<u32x4*>(a.out + p * a.pieceStride + first + within * 16) = v;
        }
    } else if (acc == 0x7fffffffu) {
        *reinterpret_cast<uint32_t*>(a.out) = acc;  // keeps the loads alive; the value never occurs
    }
}

__global__ __launch_bounds__(kThreads) void probeCopy(u32x4* __restrict__ dst, const u32x4* __restrict__ src, int64_t packets) {
    // four packets a thread in flight, each instruction of the work-group on 4 KiB of consecutive bytes; whole groups of four
    // without a branch around a load, the rest one by one
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads * 4;
    int64_t p0 = static_cast<int64_t>(blockIdx.x) * kThreads * 4 + threadIdx.x;
    for (; p0 + 3 * kThreads < packets; p0 += stride) {
        u32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(src + p0 + u * kThreads);
#pragma unroll
        for (int u = 0; u < 4; ++u) __builtin_nontemporal_store(v[u], dst + p0 + u * kThreads);
    }
    for (int u = 0; u < 4; ++u) {
        const int64_t p = p0 + u * kThreads;
        if (p < packets) dst[p] = src[p];
    }
}

// The rate the matrix cores sustain: every wave runs `iters` rounds of 16 v_mfma_f32_32x32x16 products (four accumulators,
// operands held in registers) and leaves its shader-clock and 100 MHz-clock counts behind, so that the caller gets both the
// product rate and the clock the part ran at.
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

template <bool BF16>
__global__ __launch_bounds__(512) void probeMatrixRate(long long* __restrict__ clocks, float* __restrict__ sink, int iters) {
    const int lane = threadIdx.x % 64;
    // operands: every 16-bit element gets a hashed sign and mantissa and an exponent that puts it in 1/32 .. 1/2 (the spread
    // of attention operands: scaled queries and keys, probabilities), so that consecutive products, which take different
    // operand registers, switch the multiplier inputs the way real data does
    u32x4 raw[8];
    for (int i = 0; i < 8; ++i) {
        for (int c = 0; c < 4; ++c) {
            uint32_t h = (static_cast<uint32_t>(lane) * 8u + i) * 4u + c;
            h = (h ^ 61u) ^ (h >> 16);
            h *= 9u;
            h ^= h >> 4;
            h *= 0x27d4eb2du;
            h ^= h >> 15;
            uint32_t lo, hi;
            if (BF16) {
                lo = (h & 0x807fu) | ((0x7au + ((h >> 8) & 3u)) << 7);
                hi = ((h >> 16) & 0x807fu) | ((0x7au + ((h >> 24) & 3u)) << 7);
            } else {
                lo = (h & 0x83ffu) | ((0x0au + ((h >> 11) & 3u)) << 10);
                hi = ((h >> 16) & 0x83ffu) | ((0x0au + ((h >> 27) & 3u)) << 10);
            }
            raw[i][c] = lo | (hi << 16);
        }
    }
    f32x16 acc[4];
    for (int j = 0; j < 4; ++j)
        for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
    const long long c0 = __builtin_amdgcn_s_memtime();
    const long long w0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int st = 0; st < 4; ++st) {
                const int ia = (st + j) % 8, ib = (st + 2 * j + 4) % 8;
                if constexpr (BF16) {
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, raw[ia]), __builtin_bit_cast(bf16x8, raw[ib]), acc[j], 0, 0, 0);
                } else {
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, raw[ia]), __builtin_bit_cast(f16x8, raw[ib]), acc[j], 0, 0, 0);
                }
            }
        }
    }
    const long long c1 = __builtin_amdgcn_s_memtime();
    const long long w1 = __builtin_amdgcn_s_memrealtime();
    float t = 0.f;
    for (int j = 0; j < 4; ++j)
        for (int r = 0; r < 16; ++r) t += acc[j][r];
    if (t == 1.2345f) *sink = t;
    if (lane == 0) {
        long long* c = clocks + (static_cast<long long>(blockIdx.x) * (blockDim.x / 64) + threadIdx.x / 64) * 2;
        c[0] = c1 - c0;
        c[1] = w1 - w0;
    }
}

}  // namespace

// One launch of the matrix-rate probe: `workGroups` groups of `waves` waves (4 or 8: one or two per SIMD), `iters` rounds of
// 16 products per wave.  clocks: [workGroups * waves][2] (shader clocks, 10 ns ticks) per wave; sink: 4 bytes.
extern "C" int diopiProbeMatrixRate(void* stream, void* clocks, void* sink, int workGroups, int waves, int iters, int bf16) {
    if (workGroups <= 0 || (waves != 4 && waves != 8) || iters <= 0) return 1;
    if (bf16) {
        hipLaunchKernelGGL(probeMatrixRate<true>, dim3(static_cast<unsigned>(workGroups)), dim3(static_cast<unsigned>(waves * 64)), 0,
                           static_cast<hipStream_t>(stream), static_cast<long long*>(clocks), static_cast<float*>(sink), iters);
    } else {
        hipLaunchKernelGGL(probeMatrixRate<false>, dim3(static_cast<unsigned>(workGroups)), dim3(static_cast<unsigned>(waves * 64)), 0,
                           static_cast<hipStream_t>(stream), static_cast<long long*>(clocks), static_cast<float*>(sink), iters);
    }
    return hipGetLastError() == hipSuccess ? 0 : 1;
}

// Launches one pass of the gather probe on `stream`.  Returns 0, or 1 when the arguments do not fit what the kernel assumes.
extern "C" int diopiProbeTokenGather(void* stream, int mode, const void* cache, int rowBytes, const int32_t* loc, int maxInputLen, const int32_t* start,
                                     const int32_t* length, int batch, int maxLength, void* out, int64_t pieceStride, int pieces, int bytesPerToken,
                                     int tileTokens, int rowSplit) {
    if (rowSplit <= 0 || rowBytes % rowSplit != 0) return 1;
    const int partBytes = rowBytes / rowSplit;
    const bool rowOk = partBytes >= 16 && partBytes <= 16 * kThreads && (partBytes & (partBytes - 1)) == 0;
    if (!rowOk || (mode & 3) == 0 || mode > 15 || batch <= 0 || batch > 65535 || maxLength <= 0 || tileTokens <= 0 || pieces <= 0 || bytesPerToken % pieces != 0 ||
        (tileTokens * (bytesPerToken / pieces)) % 16 != 0 || pieceStride % 16 != 0)
        return 1;
    GatherArgs a;
    a.cache = static_cast<const char*>(cache);
    a.loc = loc;
    a.start = start;
    a.length = length;
    a.out = static_cast<char*>(out);
    a.pieceStride = pieceStride;
    a.rowBytes = rowBytes;
    a.partBytes = partBytes;
    a.maxInputLen = maxInputLen;
    a.tileTokens = tileTokens;
    a.pieces = pieces;
    a.bytesPerToken = bytesPerToken;
    a.mode = mode;
    const dim3 grid(static_cast<unsigned>(rowSplit), static_cast<unsigned>(batch), static_cast<unsigned>((maxLength + tileTokens - 1) / tileTokens));
    if (tileTokens > 8192) return 1;  // the slots of a tile in LDS
    const size_t lds = static_cast<size_t>(tileTokens) * sizeof(int32_t);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (mode & 8) {
        if (mode & 4) {
            hipLaunchKernelGGL((probeTokenGather<true, 1>), grid, dim3(kThreads), lds, s, a);
        } else {
            hipLaunchKernelGGL((probeTokenGather<false, 1>), grid, dim3(kThreads), lds, s, a);
        }
    } else if (mode & 4) {
        hipLaunchKernelGGL((probeTokenGather<true, 8>), grid, dim3(kThreads), lds, s, a);
    } else {
        hipLaunchKernelGGL((probeTokenGather<false, 8>), grid, dim3(kThreads), lds, s, a);
    }
    return hipGetLastError() == hipSuccess ? 0 : 1;
}

// A plain copy of `bytes` bytes (a multiple of 16) with 16-byte accesses: the yardstick the counters and the stream rates are
// read against.
extern "C" int diopiProbeCopy(void* stream, void* dst, const void* src, int64_t bytes, int workGroups) {
    if (bytes <= 0 || bytes % 16 != 0 || workGroups <= 0) return 1;
    hipLaunchKernelGGL(probeCopy, dim3(static_cast<unsigned>(workGroups)), dim3(kThreads), 0, static_cast<hipStream_t>(stream), static_cast<u32x4*>(dst),
                       static_cast<const u32x4*>(src), bytes / 16);
    return hipGetLastError() == hipSuccess ? 0 : 1;
}
