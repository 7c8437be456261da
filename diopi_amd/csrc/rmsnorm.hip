// diopiRMSNorm / diopiRMSNormBackward for gfx950.
//
// Arithmetic follows the reference kernels in
// impl/torch/functions/functions_ext/layer_norm_cuda_kernel.cu (cuApplyRMSNorm 321-378,
// cuComputePartGradGammaBeta 451-518, cuComputeGradGammaBeta 520-570, cuComputeGradInput 572-717)
// and the host wrappers in rmsnorm.cu:17-28, 85-108 and functions_ext.cpp:66-107:
//
//   n2 = prod(normalized_shape), n1 = numel / n2
//   inv_rms[r] = rsqrt(sum_l x[r,l]^2 / n2 + eps)            accumulated in fp32 (fp64 for fp64 input)
//   out[r,l]   = weight[l] * OutT(inv_rms[r] * x[r,l])       (+ bias[l], rounded again)
//   g = dout * weight;  s[r] = sum_l g * x * inv_rms
//   grad_input[r,l]  = (inv_rms / n2) * (n2 * g - x * inv_rms * s[r])
//   grad_weight[l]   = sum_r dout[r,l] * x[r,l] * inv_rms[r]
//   grad_bias[l]     = sum_r dout[r,l]
//
// Where this design departs from the reference's launch shapes (one 128-thread block per row with
// scalar loads; grad_weight from a second full pass over x and dout):
//  * forward: one 64-lane wavefront owns a row, holds it in registers as 16-byte packets, reduces
//    with cross-lane shuffles only (no LDS, no barrier) and streams it back out: exactly one read
//    and one write of the matrix.  The weight packets stay in registers across the rows a wave
//    visits.
//  * backward: one pass.  A 256-thread group walks rows; each thread keeps the columns it owns in
//    registers for x and dout, the row sum s[r] is a single barrier away, and the column sums for
//    grad_weight / grad_bias accumulate in registers across rows.  Per-group partial sums go to a
//    context-owned scratch buffer and a small second kernel folds them.  x and dout are read once.
//  * column sums are accumulated in fp64 when the data is fp32/fp64, which makes grad_weight
//    independent of the summation order to well below fp32 rounding.
#include <type_traits>

#include "common.hpp"
#include "device.hpp"

namespace rocm {
namespace {

// ---------------------------------------------------------------------------
// Forward, register-resident row: requires n2 * sizeof(TIn) to be a multiple of 16 bytes and at
// most NV * 64 packets per row.
// ---------------------------------------------------------------------------
constexpr int kFwdThreads = 256;
constexpr int kFwdWaves = kFwdThreads / kWave;

template <typename TIn, typename TOut, int NV, bool HAS_BIAS>
__global__ __launch_bounds__(kFwdThreads) void rmsNormFwdRowReg(TOut* __restrict__ out, float* __restrict__ invRms, const TIn* __restrict__ x,
                                                                 const TOut* __restrict__ weight, const TOut* __restrict__ bias, int64_t n1, int n2,
                                                                 float eps, int rowsPerWave) {
    constexpr int EPV = Pack16<TIn>::N;  // elements per input packet
    const int lane = threadIdx.x % kWave;
    const int64_t waveId = static_cast<int64_t>(blockIdx.x) * kFwdWaves + threadIdx.x / kWave;
    const int nvec = n2 / EPV;
    int64_t row = waveId * rowsPerWave;
    int64_t rowEnd = row + rowsPerWave;
    if (rowEnd > n1) rowEnd = n1;
    if (row >= rowEnd) return;

    // weight (and bias) for the columns this lane owns, as fp32
    float w[NV][EPV];
    float b[NV][EPV];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int v = j * kWave + lane;
        if (v < nvec) {
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                w[j][e] = toFloat(weight[v * EPV + e]);
                if (HAS_BIAS) b[j][e] = toFloat(bias[v * EPV + e]);
            }
        }
    }

    const float rn2 = 1.0f / static_cast<float>(n2);
    for (; row < rowEnd; ++row) {
        const TIn* xr = x + row * n2;
        TOut* orow = out + row * n2;
        Pack16<TIn> xv[NV];
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int v = j * kWave + lane;
            if (v < nvec) xv[j] = loadPackStream(xr + v * EPV);
        }
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int v = j * kWave + lane;
            if (v < nvec) {
#pragma unroll
                for (int e = 0; e < EPV; ++e) {
                    const float f = toFloat(xv[j].e[e]);
                    ss += f * f;
                }
            }
        }
        ss = waveSum(ss);
        const float inv = 1.0f / sqrtf(ss * rn2 + eps);
        if (lane == 0) invRms[row] = inv;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int v = j * kWave + lane;
            if (v < nvec) {
                TOut o[EPV];
#pragma unroll
                for (int e = 0; e < EPV; ++e) {
                    const TOut normed = fromFloat<TOut>(inv * toFloat(xv[j].e[e]));
                    TOut r = fromFloat<TOut>(w[j][e] * toFloat(normed));
                    if (HAS_BIAS) r = fromFloat<TOut>(toFloat(r) + b[j][e]);
                    o[e] = r;
                }
                // EPV output elements are EPV*sizeof(TOut) contiguous bytes: 16, or 8 when fp32 -> 16-bit
                if constexpr (sizeof(TOut) == sizeof(TIn)) {
                    Pack16<TOut> pv;
#pragma unroll
                    for (int e = 0; e < EPV; ++e) pv.e[e] = o[e];
                    storePackStream(orow + v * EPV, pv);
                } else {
#pragma unroll
                    for (int e = 0; e < EPV; ++e) orow[v * EPV + e] = o[e];
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Forward for long rows (more than two packets per lane of a wave): a 256-thread group owns a row, each
// thread NVT packets of it; the sum of squares crosses the four waves through LDS (one barrier per
// row).  Many short-lived groups, each touching one contiguous run of rows, is the launch shape the
// memory system sustains the highest bandwidth for.
// ---------------------------------------------------------------------------
template <typename TIn, typename TOut, int NVT, bool HAS_BIAS>
__global__ __launch_bounds__(kFwdThreads) void rmsNormFwdBlockRow(TOut* __restrict__ out, float* __restrict__ invRms, const TIn* __restrict__ x,
                                                                   const TOut* __restrict__ weight, const TOut* __restrict__ bias, int64_t n1, int n2,
                                                                   float eps, int rowsPerBlock) {
    constexpr int EPV = Pack16<TIn>::N;
    __shared__ float red[2][kFwdWaves];
    const int tid = threadIdx.x;
    const int lane = tid % kWave;
    const int wave = tid / kWave;
    const int nvec = n2 / EPV;
    int64_t row = static_cast<int64_t>(blockIdx.x) * rowsPerBlock;
    int64_t rowEnd = row + rowsPerBlock;
    if (rowEnd > n1) rowEnd = n1;

    float w[NVT][EPV];
    float b[NVT][EPV];
#pragma unroll
    for (int j = 0; j < NVT; ++j) {
        const int v = j * kFwdThreads + tid;
        if (v < nvec) {
            if constexpr (sizeof(TOut) == sizeof(TIn)) {
                const Pack16<TOut> wp = loadPack(weight + v * EPV);
#pragma unroll
                for (int e = 0; e < EPV; ++e) w[j][e] = toFloat(wp.e[e]);
                if (HAS_BIAS) {
                    const Pack16<TOut> bp = loadPack(bias + v * EPV);
#pragma unroll
                    for (int e = 0; e < EPV; ++e) b[j][e] = toFloat(bp.e[e]);
                }
            } else {
#pragma unroll
                for (int e = 0; e < EPV; ++e) {
                    w[j][e] = toFloat(weight[v * EPV + e]);
                    if (HAS_BIAS) b[j][e] = toFloat(bias[v * EPV + e]);
                }
            }
        }
    }
    const float rn2 = 1.0f / static_cast<float>(n2);
    int parity = 0;
    for (; row < rowEnd; ++row, parity ^= 1) {
        const TIn* xr = x + row * n2;
        TOut* orow = out + row * n2;
        Pack16<TIn> xv[NVT];
#pragma unroll
        for (int j = 0; j < NVT; ++j) {
            const int v = j * kFwdThreads + tid;
            if (v < nvec) xv[j] = loadPackStream(xr + v * EPV);
        }
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < NVT; ++j) {
            const int v = j * kFwdThreads + tid;
            if (v < nvec) {
#pragma unroll
                for (int e = 0; e < EPV; ++e) {
                    const float f = toFloat(xv[j].e[e]);
                    ss += f * f;
                }
            }
        }
        ss = waveSum(ss);
        if (lane == 0) red[parity][wave] = ss;
        __syncthreads();
        float tot = 0.f;
#pragma unroll
        for (int i = 0; i < kFwdWaves; ++i) tot += red[parity][i];
        const float inv = 1.0f / sqrtf(tot * rn2 + eps);
        if (tid == 0) invRms[row] = inv;
#pragma unroll
        for (int j = 0; j < NVT; ++j) {
            const int v = j * kFwdThreads + tid;
            if (v < nvec) {
                TOut o[EPV];
#pragma unroll
                for (int e = 0; e < EPV; ++e) {
                    const TOut normed = fromFloat<TOut>(inv * toFloat(xv[j].e[e]));
                    TOut r = fromFloat<TOut>(w[j][e] * toFloat(normed));
                    if (HAS_BIAS) r = fromFloat<TOut>(toFloat(r) + b[j][e]);
                    o[e] = r;
                }
                if constexpr (sizeof(TOut) == sizeof(TIn)) {
                    Pack16<TOut> pv;
#pragma unroll
                    for (int e = 0; e < EPV; ++e) pv.e[e] = o[e];
                    storePackStream(orow + v * EPV, pv);
                } else {
#pragma unroll
                    for (int e = 0; e < EPV; ++e) orow[v * EPV + e] = o[e];
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Forward, any shape / dtype combination: one wavefront per row, two sweeps over the row
// (the second one hits in cache).  AccT is float or double.
// ---------------------------------------------------------------------------
template <typename TIn, typename TOut, typename AccT>
__global__ __launch_bounds__(kFwdThreads) void rmsNormFwdGeneric(TOut* __restrict__ out, AccT* __restrict__ invRms, const TIn* __restrict__ x,
                                                                  const TOut* __restrict__ weight, const TOut* __restrict__ bias, int64_t n1, int64_t n2,
                                                                  AccT eps) {
    const int lane = threadIdx.x % kWave;
    const int64_t wavesTotal = static_cast<int64_t>(gridDim.x) * kFwdWaves;
    for (int64_t row = static_cast<int64_t>(blockIdx.x) * kFwdWaves + threadIdx.x / kWave; row < n1; row += wavesTotal) {
        const TIn* xr = x + row * n2;
        TOut* orow = out + row * n2;
        AccT ss = 0;
        for (int64_t l = lane; l < n2; l += kWave) {
            const AccT f = static_cast<AccT>(xr[l]);
            ss += f * f;
        }
        ss = waveSum(ss);
        AccT inv;
        if constexpr (sizeof(AccT) == 8) {
            inv = 1.0 / sqrt(ss / static_cast<AccT>(n2) + eps);
        } else {
            inv = 1.0f / sqrtf(ss / static_cast<AccT>(n2) + eps);
        }
        if (lane == 0) invRms[row] = inv;
        for (int64_t l = lane; l < n2; l += kWave) {
            const TOut normed = static_cast<TOut>(inv * static_cast<AccT>(xr[l]));
            // the product of two OutT values is formed in the accumulation type and rounded once
            TOut r = static_cast<TOut>(static_cast<AccT>(weight[l]) * static_cast<AccT>(normed));
            if (bias != nullptr) r = static_cast<TOut>(static_cast<AccT>(r) + static_cast<AccT>(bias[l]));
            orow[l] = r;
        }
    }
}

// ---------------------------------------------------------------------------
// Backward, fused single pass (T = dtype of x, dout, weight, grad_input, grad_weight).
// A work-group is GROUPS row teams of TEAM threads (256, 512 or 1024: the launcher says when), one work-group per compute
// unit.  In step i, team g of work-group b takes row
// (i * gridDim.x + b) * GROUPS + g: at any moment the whole grid works on one contiguous window of
// gridDim.x * GROUPS rows of each tensor, which spreads the traffic evenly over the memory channels (a private run of
// rows per work-group would put the work-groups, which advance in step, a fixed large stride apart).
// Thread t of a team owns packets t, t+TEAM, ... of every row its team visits.
//
// Rows travel through buffer loads and stores whose descriptor covers exactly one row (and nothing for a row past
// the end of the work-group's run): packets beyond the row read as zero and stores to them are dropped by the
// hardware, so the row loop has no branch around a memory instruction.  A team keeps two rows in registers: while
// the row of step i is reduced and written back, the row of step i+1 is already there and the row of step i+2 is
// requested into the registers the first one leaves.  The first step is peeled off the loop so that every later step sees the same sequence of
// outstanding memory operations (one row of loads, the stores of the previous step, the next row of loads) and only
// waits for the oldest of them.
//
// The column sums for grad_weight / grad_bias are accumulated in fp32 registers and moved every kBwdFlush steps into
// per-team LDS arrays of ColAcc (fp64 for fp32 tensors), which bounds the length of any fp32 summation; at the end
// the team arrays are summed in a fixed order into one fp32 partial row per work-group (one rounding of a sum that the
// fold then continues in fp64: the error stays below one rounding of the fp32 result).  The fewer packets of a row a thread
// holds, the faster the rows stream: at fp32 [8192, 4096] one work-group of four 256-thread teams (4 packets a thread)
// moves the rows at 5.79 TB/s, two work-groups of two such teams per unit at 6.07, one work-group of two 512-thread teams
// (2 packets a thread, one partial row per unit) is another 2.5 % faster over the whole operator and one team of 1024
// threads (1 packet a thread) 2 % more.  The row sum s[r] crosses the team's waves through LDS: one barrier per step.
// ---------------------------------------------------------------------------
constexpr int kBwdTeam = 256;  // threads of a team unless a shape asks for more
constexpr int kBwdFlush = 8;
constexpr int kBufferWord3 = 0x00020000;  // raw buffer, 32-bit data format
constexpr int kBufferStream = 2;          // cache policy: non-temporal

template <typename T>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t rowBuffer(const T* base, int64_t row, int n2, bool valid) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(base + row * n2), 0, valid ? n2 * static_cast<int>(sizeof(T)) : 0, kBufferWord3);
}

// A work-group is GROUPS teams of TEAM threads (256 or 512), one work-group per compute unit: GROUPS * TEAM / 256 waves on
// each of its four SIMDs, which is what the second launch bound states (and what sets the registers a lane may use).
template <typename T, typename ColAcc, int NVT, bool HAS_GBIAS, int GROUPS, int TEAM>
__global__ __launch_bounds__(TEAM* GROUPS, GROUPS*(TEAM / 256)) void rmsNormBwdFused(T* __restrict__ gradInput, float* __restrict__ partW, float* __restrict__ partB,
                                                                       const T* __restrict__ dout, const T* __restrict__ x, const T* __restrict__ weight,
                                                                       const float* __restrict__ invRms, int64_t n1, int n2) {
    constexpr int EPV = Pack16<T>::N;
    constexpr int kCols = NVT * TEAM * EPV;  // columns covered by the register tiling
    __shared__ float red[2][GROUPS][(TEAM / kWave)];
    extern __shared__ __attribute__((aligned(16))) unsigned char dynLds[];
    // [array(W,B)][team][(j*EPV + e)][tid]: lanes of a wave hit consecutive words
    ColAcc* sAcc = reinterpret_cast<ColAcc*>(dynLds);
    const int team = __builtin_amdgcn_readfirstlane(threadIdx.x / TEAM);  // the same for all lanes of a wave
    const int tid = threadIdx.x % TEAM;
    const int lane = tid % kWave;
    const int wave = tid / kWave;
    ColAcc* myW = sAcc + team * kCols;
    ColAcc* myB = sAcc + (GROUPS + team) * kCols;

    const int64_t rowsPerStep = static_cast<int64_t>(gridDim.x) * GROUPS;
    const int steps = static_cast<int>((n1 + rowsPerStep - 1) / rowsPerStep);  // the same for every work-group
    auto rowOf = [&](int i) { return (static_cast<int64_t>(i) * gridDim.x + blockIdx.x) * GROUPS + team; };

    struct RowRegs {
        Pack16<T> x[NVT], d[NVT];
        float inv;
    };
    auto request = [&](RowRegs& r, int64_t row) {
        const bool valid = row < n1;
        const __amdgpu_buffer_rsrc_t bx = rowBuffer(x, row, n2, valid);
        const __amdgpu_buffer_rsrc_t bd = rowBuffer(dout, row, n2, valid);
#pragma unroll
        for (int j = 0; j < NVT; ++j) {
            const int off = (j * TEAM + tid) * 16;
            r.x[j].raw = __builtin_amdgcn_raw_buffer_load_b128(bx, off, 0, kBufferStream);
            r.d[j].raw = __builtin_amdgcn_raw_buffer_load_b128(bd, off, 0, kBufferStream);
        }
        r.inv = invRms[valid ? row : 0];  // uniform address: a scalar load, no branch
    };

    // the weight packets are requested before the rows: a wait for the first row then covers them as well
    Pack16<T> wv[NVT];
    {
        const __amdgpu_buffer_rsrc_t bw = rowBuffer(weight, 0, n2, true);
#pragma unroll
        for (int j = 0; j < NVT; ++j) wv[j].raw = __builtin_amdgcn_raw_buffer_load_b128(bw, (j * TEAM + tid) * 16, 0, 0);
    }
    RowRegs ra, rb;
    request(ra, rowOf(0));
    request(rb, rowOf(1));

    float w[NVT][EPV], accW[NVT][EPV], accB[HAS_GBIAS ? NVT : 1][EPV];
    {
#pragma unroll
        for (int j = 0; j < NVT; ++j) {
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                w[j][e] = toFloat(wv[j].e[e]);
                accW[j][e] = 0.f;
                if (HAS_GBIAS) accB[j][e] = 0.f;
                myW[(j * EPV + e) * TEAM + tid] = 0;
                if (HAS_GBIAS) myB[(j * EPV + e) * TEAM + tid] = 0;
            }
        }
    }
    // registers -> this team's LDS arrays; each (team, column) word has exactly one writer
    auto flush = [&]() {
#pragma unroll
        for (int j = 0; j < NVT; ++j) {
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                myW[(j * EPV + e) * TEAM + tid] += static_cast<ColAcc>(accW[j][e]);
                accW[j][e] = 0.f;
                if (HAS_GBIAS) {
                    myB[(j * EPV + e) * TEAM + tid] += static_cast<ColAcc>(accB[j][e]);
                    accB[j][e] = 0.f;
                }
            }
        }
    };

    const float fH = static_cast<float>(n2);
    // One row step of a team on the registers r; rows past the end arrive as zeros and their stores are dropped.
    auto step = [&](RowRegs& r, int i) {
        const int64_t row = rowOf(i);
        const float inv = r.inv;
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < NVT; ++j) {
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                const float cx = toFloat(r.x[j].e[e]);
                const float cd = toFloat(r.d[j].e[e]);
                s += cd * w[j][e] * cx * inv;
                accW[j][e] += cd * cx * inv;
                if (HAS_GBIAS) accB[j][e] += cd;
            }
        }
        s = waveSum(s);
        if (lane == 0) red[i & 1][team][wave] = s;
        __syncthreads();
        float sum2 = 0.f;
#pragma unroll
        for (int k = 0; k < (TEAM / kWave); ++k) sum2 += red[i & 1][team][k];
        const float term1 = (1.0f / fH) * inv;
        const __amdgpu_buffer_rsrc_t bg = rowBuffer(gradInput, row, n2, row < n1);
#pragma unroll
        for (int j = 0; j < NVT; ++j) {
            Pack16<T> gv;
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                const float cx = toFloat(r.x[j].e[e]);
                const float cd = toFloat(r.d[j].e[e]);
                float f = fH * cd * w[j][e];
                f -= cx * inv * sum2;
                f *= term1;
                gv.e[e] = fromFloat<T>(f);
            }
            __builtin_amdgcn_raw_buffer_store_b128(gv.raw, bg, (j * TEAM + tid) * 16, 0, kBufferStream);
        }
        request(r, rowOf(i + 2));
        if ((i % kBwdFlush) == kBwdFlush - 1) flush();
    };

    step(ra, 0);  // n1 > 0: there is at least one step
    // whole pairs in the loop (no exit between the two halves, so both see one fixed sequence of outstanding operations)
    int i = 1;
    for (; i + 1 < steps; i += 2) {
        step(rb, i);
        step(ra, i + 1);
    }
    if (i < steps) step(rb, i);
    if (steps % kBwdFlush != 0) flush();  // what the last steps left in registers

    // one partial row per work-group: the team arrays are added in team order
    __syncthreads();
    for (int idx = threadIdx.x; idx < kCols; idx += TEAM * GROUPS) {
        // idx = (j*EPV + e)*256 + t  <->  column (j*256 + t)*EPV + e
        const int t = idx % TEAM;
        const int je = idx / TEAM;
        const int col = ((je / EPV) * TEAM + t) * EPV + (je % EPV);
        if (col < n2) {
            ColAcc sw = 0, sb = 0;
#pragma unroll
            for (int g = 0; g < GROUPS; ++g) {
                sw += sAcc[g * kCols + idx];
                if (HAS_GBIAS) sb += sAcc[(GROUPS + g) * kCols + idx];
            }
            partW[static_cast<int64_t>(blockIdx.x) * n2 + col] = static_cast<float>(sw);
            if (HAS_GBIAS) partB[static_cast<int64_t>(blockIdx.x) * n2 + col] = static_cast<float>(sb);
        }
    }
}

// Folds the [numParts, n2] fp32 partial rows into grad_weight (and grad_bias) in fp64.  A 256-thread group covers 32
// consecutive columns (8 threads x 16 bytes = 128 bytes of a partial row) x 32 slices of the rows; a thread's loads of a
// batch are independent and in flight together, so 512 partial rows are one round trip.  n2 is a multiple of 4.
constexpr int kFoldCols = 32;  // 16 and 64 columns per group measured 1.3 us slower at 512 partial rows of 4096
constexpr int kFoldSlices = 256 / (kFoldCols / 4);
template <typename T>
__global__ __launch_bounds__(256) void rmsNormBwdFold(T* __restrict__ gradWeight, T* __restrict__ gradBias, const float* __restrict__ partW,
                                                       const float* __restrict__ partB, int numParts, int n2) {
    __shared__ double red[2][kFoldSlices][kFoldCols + 1];
    const int c4 = threadIdx.x % (kFoldCols / 4);
    const int slice = threadIdx.x / (kFoldCols / 4);
    const int col = blockIdx.x * kFoldCols + c4 * 4;
    double sw[4] = {0.0, 0.0, 0.0, 0.0}, sb[4] = {0.0, 0.0, 0.0, 0.0};
    if (col < n2) {
        constexpr int kBatch = 16;
        const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
        for (int p0 = slice; p0 < numParts; p0 += kFoldSlices * kBatch) {
            f32x4 vw[kBatch], vb[kBatch];
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                const int p = p0 + kFoldSlices * u;
                vw[u] = p < numParts ? *reinterpret_cast<const f32x4*>(partW + static_cast<int64_t>(p) * n2 + col) : zero;
                vb[u] = (gradBias != nullptr && p < numParts) ? *reinterpret_cast<const f32x4*>(partB + static_cast<int64_t>(p) * n2 + col) : zero;
            }
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    sw[e] += static_cast<double>(vw[u][e]);
                    sb[e] += static_cast<double>(vb[u][e]);
                }
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        red[0][slice][c4 * 4 + e] = sw[e];
        red[1][slice][c4 * 4 + e] = sb[e];
    }
    __syncthreads();
    // threads 0..31 finish grad_weight, 32..63 grad_bias: the slices in their fixed order
    const int which = threadIdx.x / kFoldCols;
    const int c = threadIdx.x % kFoldCols;
    const int outCol = blockIdx.x * kFoldCols + c;
    if (which < 2 && outCol < n2 && (which == 0 || gradBias != nullptr)) {
        double sum = 0.0;
#pragma unroll 8
        for (int k = 0; k < kFoldSlices; ++k) sum += red[which][k][c];
        (which == 0 ? gradWeight : gradBias)[outCol] = fromDouble<T>(sum);
    }
}

// ---------------------------------------------------------------------------
// Backward, any shape / dtype combination (TX: x and grad_input; TV: dout, weight, grad_weight).
// ---------------------------------------------------------------------------
template <typename TX, typename TV, typename AccT>
__global__ __launch_bounds__(kFwdThreads) void rmsNormBwdInputGeneric(TX* __restrict__ gradInput, const TV* __restrict__ dout, const TX* __restrict__ x,
                                                                       const TV* __restrict__ weight, const AccT* __restrict__ invRms, int64_t n1,
                                                                       int64_t n2) {
    const int lane = threadIdx.x % kWave;
    const int64_t wavesTotal = static_cast<int64_t>(gridDim.x) * kFwdWaves;
    for (int64_t row = static_cast<int64_t>(blockIdx.x) * kFwdWaves + threadIdx.x / kWave; row < n1; row += wavesTotal) {
        const TX* xr = x + row * n2;
        const TV* dr = dout + row * n2;
        const AccT inv = invRms[row];
        AccT s = 0;
        for (int64_t l = lane; l < n2; l += kWave) {
            s += static_cast<AccT>(dr[l]) * static_cast<AccT>(weight[l]) * static_cast<AccT>(xr[l]) * inv;
        }
        s = waveSum(s);
        const AccT fH = static_cast<AccT>(n2);
        const AccT term1 = (static_cast<AccT>(1) / fH) * inv;
        for (int64_t l = lane; l < n2; l += kWave) {
            AccT f = fH * static_cast<AccT>(dr[l]) * static_cast<AccT>(weight[l]);
            f -= static_cast<AccT>(xr[l]) * inv * s;
            f *= term1;
            gradInput[row * n2 + l] = static_cast<TX>(f);
        }
    }
}

// One thread per column, rows walked in order; the products are formed in AccT and summed in fp64.
template <typename TX, typename TV, typename AccT>
__global__ __launch_bounds__(256) void rmsNormBwdWeightGeneric(TV* __restrict__ gradWeight, TV* __restrict__ gradBias, const TV* __restrict__ dout,
                                                                const TX* __restrict__ x, const AccT* __restrict__ invRms, int64_t n1, int64_t n2) {
    const int64_t col = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (col >= n2) return;
    double sw = 0.0, sb = 0.0;
    for (int64_t r = 0; r < n1; ++r) {
        const AccT cd = static_cast<AccT>(dout[r * n2 + col]);
        sw += static_cast<double>(cd * static_cast<AccT>(x[r * n2 + col]) * invRms[r]);
        sb += static_cast<double>(cd);
    }
    gradWeight[col] = fromDouble<TV>(sw);
    if (gradBias != nullptr) gradBias[col] = fromDouble<TV>(sb);
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
struct NormDims {
    int64_t n1 = 1, n2 = 1;
    int lead = 0;  // number of leading (non-normalised) dimensions
};

// Same rule as compute_n1_n2 / check_args in rmsnorm.cu:17-65 of the reference.
diopiError_t normDims(const TensorView& input, diopiSize_t normalizedShape, NormDims* dims) {
    ROCM_CHECK(normalizedShape.len >= 1 && normalizedShape.data != nullptr, "normalized_shape must have at least one dimension");
    ROCM_CHECK(normalizedShape.len <= input.ndim, "normalized_shape has rank %lld but input has rank %d", static_cast<long long>(normalizedShape.len),
               input.ndim);
    dims->lead = input.ndim - static_cast<int>(normalizedShape.len);
    dims->n1 = 1;
    dims->n2 = 1;
    for (int i = 0; i < dims->lead; ++i) dims->n1 *= input.shape[i];
    for (int i = 0; i < normalizedShape.len; ++i) {
        ROCM_CHECK(input.shape[dims->lead + i] == normalizedShape.data[i], "normalized_shape[%d] = %lld does not match input extent %lld", i,
                   static_cast<long long>(normalizedShape.data[i]), static_cast<long long>(input.shape[dims->lead + i]));
        dims->n2 *= normalizedShape.data[i];
    }
    return diopiSuccess;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// number of waves (or 256-thread groups) that are resident at once, used to size persistent launches
int residentWavesTarget() { return deviceInfo().numCU * 12; }

template <typename TIn, typename TOut>
diopiError_t launchFwdFast(hipStream_t stream, const TensorView& out, const TensorView& invRms, const TensorView& in, const TensorView& w,
                           const void* bias, const NormDims& d, double eps, bool* launched) {
    constexpr int EPV = Pack16<TIn>::N;
    *launched = false;
    if (d.n2 % EPV != 0 || d.n2 > INT32_MAX) return diopiSuccess;
    const int64_t nvec = d.n2 / EPV;
    if (nvec > 16 * kWave) return diopiSuccess;
    if (!aligned16(in.data) || !aligned16(out.data) || !aligned16(w.data) || !aligned16(bias)) return diopiSuccess;
    if (sizeof(TOut) != sizeof(TIn) && (reinterpret_cast<uintptr_t>(out.data) & 7) != 0) return diopiSuccess;
    const float feps = static_cast<float>(eps);
    const int n2 = static_cast<int>(d.n2);
    if (nvec > 2 * kWave) {
        // long rows: one 256-thread group per run of rows
        const int nvt = static_cast<int>(ceilDiv(nvec, kFwdThreads));
        const int rpb = 1;  // rows per work-group
        const unsigned gridB = static_cast<unsigned>(ceilDiv(d.n1, rpb));
#define ROCM_FWDB_CASE(NVC)                                                                                                                         \
    if (bias != nullptr) {                                                                                                                          \
        hipLaunchKernelGGL((rmsNormFwdBlockRow<TIn, TOut, NVC, true>), dim3(gridB), dim3(kFwdThreads), 0, stream, static_cast<TOut*>(out.data),      \
                           static_cast<float*>(invRms.data), static_cast<const TIn*>(in.data), static_cast<const TOut*>(w.data),                      \
                           static_cast<const TOut*>(bias), d.n1, n2, feps, rpb);                                                                      \
    } else {                                                                                                                                        \
        hipLaunchKernelGGL((rmsNormFwdBlockRow<TIn, TOut, NVC, false>), dim3(gridB), dim3(kFwdThreads), 0, stream, static_cast<TOut*>(out.data),     \
                           static_cast<float*>(invRms.data), static_cast<const TIn*>(in.data), static_cast<const TOut*>(w.data),                      \
                           static_cast<const TOut*>(nullptr), d.n1, n2, feps, rpb);                                                                   \
    }
        if (nvt <= 1) {
            ROCM_FWDB_CASE(1)
        } else if (nvt <= 2) {
            ROCM_FWDB_CASE(2)
        } else {
            ROCM_FWDB_CASE(4)
        }
#undef ROCM_FWDB_CASE
        ROCM_LAUNCH_CHECK();
        *launched = true;
        return diopiSuccess;
    }
    const int nv = static_cast<int>(ceilDiv(nvec, kWave));
    // every wave takes the same number of rows so that all of them fit on the device at once
    int rowsPerWave = static_cast<int>(ceilDiv(d.n1, residentWavesTarget()));
    if (rowsPerWave < 1) rowsPerWave = 1;
    const int64_t waves = ceilDiv(d.n1, rowsPerWave);
    const unsigned grid = static_cast<unsigned>(ceilDiv(waves, kFwdWaves));
#define ROCM_FWD_CASE(NVC)                                                                                                                          \
    if (bias != nullptr) {                                                                                                                          \
        hipLaunchKernelGGL((rmsNormFwdRowReg<TIn, TOut, NVC, true>), dim3(grid), dim3(kFwdThreads), 0, stream, static_cast<TOut*>(out.data),         \
                           static_cast<float*>(invRms.data), static_cast<const TIn*>(in.data), static_cast<const TOut*>(w.data),                      \
                           static_cast<const TOut*>(bias), d.n1, n2, feps, rowsPerWave);                                                              \
    } else {                                                                                                                                        \
        hipLaunchKernelGGL((rmsNormFwdRowReg<TIn, TOut, NVC, false>), dim3(grid), dim3(kFwdThreads), 0, stream, static_cast<TOut*>(out.data),        \
                           static_cast<float*>(invRms.data), static_cast<const TIn*>(in.data), static_cast<const TOut*>(w.data),                      \
                           static_cast<const TOut*>(nullptr), d.n1, n2, feps, rowsPerWave);                                                           \
    }
    if (nv <= 1) {
        ROCM_FWD_CASE(1)
    } else if (nv <= 2) {
        ROCM_FWD_CASE(2)
    } else if (nv <= 4) {
        ROCM_FWD_CASE(4)
    } else if (nv <= 8) {
        ROCM_FWD_CASE(8)
    } else {
        ROCM_FWD_CASE(16)
    }
#undef ROCM_FWD_CASE
    ROCM_LAUNCH_CHECK();
    *launched = true;
    return diopiSuccess;
}

template <typename TIn, typename TOut, typename AccT>
diopiError_t launchFwdGeneric(hipStream_t stream, const TensorView& out, const TensorView& invRms, const TensorView& in, const TensorView& w,
                              const void* bias, const NormDims& d, double eps) {
    int64_t blocks = ceilDiv(d.n1, kFwdWaves);
    const int64_t cap = static_cast<int64_t>(deviceInfo().numCU) * 8;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL((rmsNormFwdGeneric<TIn, TOut, AccT>), dim3(static_cast<unsigned>(blocks)), dim3(kFwdThreads), 0, stream,
                       static_cast<TOut*>(out.data), static_cast<AccT*>(invRms.data), static_cast<const TIn*>(in.data), static_cast<const TOut*>(w.data),
                       static_cast<const TOut*>(bias), d.n1, d.n2, static_cast<AccT>(eps));
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
}

template <typename TIn, typename TOut>
diopiError_t forwardTyped(hipStream_t stream, const TensorView& out, const TensorView& invRms, const TensorView& in, const TensorView& w,
                          const void* bias, const NormDims& d, double eps) {
    using AccT = typename AccType<TIn>::type;
    if constexpr (sizeof(AccT) == 4 && sizeof(TIn) >= sizeof(TOut)) {
        bool launched = false;
        ROCM_CALL((launchFwdFast<TIn, TOut>(stream, out, invRms, in, w, bias, d, eps, &launched)));
        if (launched) return diopiSuccess;
    }
    return launchFwdGeneric<TIn, TOut, AccT>(stream, out, invRms, in, w, bias, d, eps);
}

// Launches one instantiation of the fused backward kernel; the LDS column-sum arrays are dynamic shared memory
// beyond the 64 KiB static limit, which has to be granted per kernel and device.
template <typename T, typename ColAcc, int NVT, bool GB, int GROUPS, int TEAM = kBwdTeam>
diopiError_t launchBwdInstance(hipStream_t stream, int numParts, T* gIn, float* partW, float* partB, const T* dout, const T* in, const T* w,
                               const float* invRms, int64_t n1, int n2) {
    constexpr int EPV = Pack16<T>::N;
    constexpr size_t ldsBytes = static_cast<size_t>(GB ? 2 : 1) * GROUPS * NVT * TEAM * EPV * sizeof(ColAcc);
    auto kernel = rmsNormBwdFused<T, ColAcc, NVT, GB, GROUPS, TEAM>;
    ROCM_CALL(grantDynamicLds(reinterpret_cast<const void*>(kernel), static_cast<int>(ldsBytes)));
    hipLaunchKernelGGL(kernel, dim3(numParts), dim3(TEAM * GROUPS), ldsBytes, stream, gIn, partW, partB, dout, in, w, invRms, n1, n2);
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
}

template <typename T, typename ColAcc>
diopiError_t launchBwdFused(diopiContextHandle_t ctx, hipStream_t stream, const TensorView& gIn, const TensorView& gW, void* gBias, const TensorView& dout,
                            const TensorView& in, const TensorView& w, const TensorView& invRms, const NormDims& d, bool* launched) {
    constexpr int EPV = Pack16<T>::N;
    *launched = false;
    if (d.n2 % EPV != 0 || d.n2 > INT32_MAX) return diopiSuccess;
    const int64_t nvec = d.n2 / EPV;
    // The shape of the work-groups by the packets a thread holds per row (NVT), all within 128 KiB of LDS per compute unit
    // (a team array is NVT * 256 packets of ColAcc).  Measured without grad_bias, main kernel alone:
    //   fp32 [8192, 4096] (NVT 4): two groups of two teams 68.0 us, one group of four teams 71.4 us
    //   fp32 [32768, 1024] (NVT 1): 67.5 against 63.4 us; bf16 [8192, 4096] (NVT 2): 37.8 against 36.7 us
    //   bf16 [4096, 8192] (NVT 4): one group of two teams 46.3 us against 108.9 us for four teams, whose 16 waves leave a lane
    //   128 registers where the kernel wants 217
    // so fewer packets than four take one group of four teams; 16-bit NVT 4 (217 registers) and fp32 rows of up to 8192 columns
    // (NVT 8, 64 KiB per team array, 236 registers) one group of two.  With grad_bias a team has two arrays: one group of two
    // teams (one of one team at NVT 8).  Wider teams where they pay: see below.
    constexpr int kMaxNvt = sizeof(T) == 4 ? 8 : 4;
    if (nvec > static_cast<int64_t>(kMaxNvt) * kBwdTeam) return diopiSuccess;
    if (deviceInfo().maxSharedOptin < 128 * 1024 + 1024) return diopiSuccess;
    if (!aligned16(in.data) || !aligned16(dout.data) || !aligned16(gIn.data) || !aligned16(w.data)) return diopiSuccess;
    const int nvt = static_cast<int>(ceilDiv(nvec, kBwdTeam));
    const int nvc = nvt <= 1 ? 1 : (nvt <= 2 ? 2 : (nvt <= 4 ? 4 : 8));
    // The fewer packets of a row a thread holds, the faster the rows stream.  With at least 16 rows per compute unit and no
    // grad_bias, rows of more than 256 packets therefore go to the widest team they fill, 1024 threads in all (us, teams of
    // 256 threads as above -> wide teams):
    //   fp32 [8192, 4096] 71.7 -> 68.6 (two teams of 512: 69.9), [16384, 4096] 137.0 -> 130.2, [4096, 8192] 78.4 -> 76.0
    //   bf16 [8192, 4096] 39.8 -> 39.3, [16384, 4096] 71.3 -> 69.5, [4096, 8192] 43.5 -> 42.9
    // With fewer rows the wide teams lose ([2048, 4096]: fp32 21.1 -> 23.3, bf16 16.0 -> 16.9: too few teams to spread the rows
    // over), and with grad_bias they change nothing (fp32 [8192, 4096] 71.0 -> 71.1) or lose (bf16 43.2 -> 43.6), except that
    // fp32 rows of 1024 packets take one team of 512 threads there (73.1 -> 70.9).
    const bool manyRows = d.n1 >= 16 * static_cast<int64_t>(deviceInfo().numCU);
    const bool wide = gBias == nullptr && manyRows && nvec > 256;
    const bool wideBias = gBias != nullptr && nvc == 4 && sizeof(T) == 4;
    // teams of a work-group: each owns rows of its own
    const int groups = wide ? (nvec <= 512 ? 2 : 1) : (wideBias ? 1 : (gBias ? (nvc == 8 ? 1 : 2) : ((nvc <= 2 || (nvc == 4 && sizeof(T) == 4)) ? 4 : 2)));
    // as many work-groups as there are compute units (fewer when there are not enough rows to give every team one)
    const int64_t maxBlocks = deviceInfo().numCU;
    const int teamsPerGroup = groups;
    const int numParts = static_cast<int>(std::min<int64_t>(maxBlocks, ceilDiv(d.n1, teamsPerGroup)));
    const int n2 = static_cast<int>(d.n2);
    const int64_t partBytes = static_cast<int64_t>(numParts) * n2 * sizeof(float);
    void* scratch = nullptr;
    ROCM_CALL(requireScratch(ctx, partBytes * (gBias ? 2 : 1), &scratch));
    float* partW = static_cast<float*>(scratch);
    float* partB = gBias ? partW + static_cast<int64_t>(numParts) * n2 : nullptr;
    T* pgi = static_cast<T*>(gIn.data);
    const T* pdo = static_cast<const T*>(dout.data);
    const T* pin = static_cast<const T*>(in.data);
    const T* pw = static_cast<const T*>(w.data);
    const float* pinv = static_cast<const float*>(invRms.data);
#define ROCM_BWD_CASE(NVC, GB, GROUPS, TEAM) \
    ROCM_CALL((launchBwdInstance<T, ColAcc, NVC, GB, GROUPS, TEAM>(stream, numParts, pgi, partW, partB, pdo, pin, pw, pinv, d.n1, n2)))
    if (wide) {
        if (nvec <= 512) {
            ROCM_BWD_CASE(1, false, 2, 512);
        } else if (nvec <= 1024) {
            ROCM_BWD_CASE(1, false, 1, 1024);
        } else if constexpr (kMaxNvt >= 8) {
            ROCM_BWD_CASE(2, false, 1, 1024);
        }
    } else if (gBias != nullptr) {
        if (nvc == 1) {
            ROCM_BWD_CASE(1, true, 2, 256);
        } else if (nvc == 2) {
            ROCM_BWD_CASE(2, true, 2, 256);
        } else if (nvc == 4) {
            if constexpr (sizeof(T) == 4) {
                ROCM_BWD_CASE(2, true, 1, 512);
            } else {
                ROCM_BWD_CASE(4, true, 2, 256);
            }
        } else if constexpr (kMaxNvt >= 8) {
            ROCM_BWD_CASE(8, true, 1, 256);
        }
    } else {
        if (nvc == 1) {
            ROCM_BWD_CASE(1, false, 4, 256);
        } else if (nvc == 2) {
            ROCM_BWD_CASE(2, false, 4, 256);
        } else if (nvc == 4) {
            if constexpr (sizeof(T) == 4) {
                ROCM_BWD_CASE(4, false, 4, 256);
            } else {
                ROCM_BWD_CASE(4, false, 2, 256);
            }
        } else if constexpr (kMaxNvt >= 8) {
            ROCM_BWD_CASE(8, false, 2, 256);
        }
    }
#undef ROCM_BWD_CASE
    hipLaunchKernelGGL((rmsNormBwdFold<T>), dim3(static_cast<unsigned>(ceilDiv(n2, kFoldCols))), dim3(256), 0, stream, static_cast<T*>(gW.data),
                       static_cast<T*>(gBias), partW, partB, numParts, n2);
    ROCM_LAUNCH_CHECK();
    *launched = true;
    return diopiSuccess;
}

template <typename TX, typename TV>
diopiError_t backwardTyped(diopiContextHandle_t ctx, hipStream_t stream, const TensorView& gIn, const TensorView& gW, void* gBias, const TensorView& dout,
                           const TensorView& in, const TensorView& w, const TensorView& invRms, const NormDims& d) {
    using AccT = typename AccType<TX>::type;
    if constexpr (std::is_same<TX, TV>::value && sizeof(AccT) == 4) {
        bool launched = false;
        if constexpr (sizeof(TX) == 4) {
            ROCM_CALL((launchBwdFused<TX, double>(ctx, stream, gIn, gW, gBias, dout, in, w, invRms, d, &launched)));
        } else {
            ROCM_CALL((launchBwdFused<TX, float>(ctx, stream, gIn, gW, gBias, dout, in, w, invRms, d, &launched)));
        }
        if (launched) return diopiSuccess;
    }
    int64_t blocks = ceilDiv(d.n1, kFwdWaves);
    const int64_t cap = static_cast<int64_t>(deviceInfo().numCU) * 8;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL((rmsNormBwdInputGeneric<TX, TV, AccT>), dim3(static_cast<unsigned>(blocks)), dim3(kFwdThreads), 0, stream,
                       static_cast<TX*>(gIn.data), static_cast<const TV*>(dout.data), static_cast<const TX*>(in.data), static_cast<const TV*>(w.data),
                       static_cast<const AccT*>(invRms.data), d.n1, d.n2);
    ROCM_LAUNCH_CHECK();
    hipLaunchKernelGGL((rmsNormBwdWeightGeneric<TX, TV, AccT>), dim3(static_cast<unsigned>(ceilDiv(d.n2, 256))), dim3(256), 0, stream,
                       static_cast<TV*>(gW.data), static_cast<TV*>(gBias), static_cast<const TV*>(dout.data), static_cast<const TX*>(in.data),
                       static_cast<const AccT*>(invRms.data), d.n1, d.n2);
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
}

// inv_rms carries the leading dimensions of the input (diopi_functions.py:7046-7054 of the reference).
diopiError_t checkInvRms(const TensorView& invRms, const TensorView& in, const NormDims& d) {
    const diopiDtype_t want = in.dtype == diopi_dtype_float64 ? diopi_dtype_float64 : diopi_dtype_float32;
    ROCM_CHECK(invRms.dtype == want, "inv_rms must be %s for %s input, got %s", dtypeName(want), dtypeName(in.dtype), dtypeName(invRms.dtype));
    ROCM_CHECK(invRms.numel == d.n1, "inv_rms has %lld elements, expected %lld (the leading dimensions of input)", static_cast<long long>(invRms.numel),
               static_cast<long long>(d.n1));
    return diopiSuccess;
}

diopiError_t checkParam(const TensorView& p, const char* name, diopiSize_t normalizedShape, diopiDtype_t dtype) {
    ROCM_CHECK(p.dtype == dtype, "%s must have dtype %s, got %s", name, dtypeName(dtype), dtypeName(p.dtype));
    ROCM_CHECK(p.ndim == normalizedShape.len, "%s must have the shape of normalized_shape", name);
    for (int i = 0; i < p.ndim; ++i) {
        ROCM_CHECK(p.shape[i] == normalizedShape.data[i], "%s must have the shape of normalized_shape", name);
    }
    return diopiSuccess;
}

}  // namespace
}  // namespace rocm

extern "C" diopiError_t diopiRMSNorm(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiTensorHandle_t inv_rms, diopiConstTensorHandle_t input,
                                     diopiSize_t normalized_shape, diopiConstTensorHandle_t weight, diopiConstTensorHandle_t bias, double eps) {
    ROCM_ENTRY_BEGIN
    using namespace rocm;
    TensorView vOut, vInv, vIn, vW, vB;
    ROCM_CALL(unwrap(out, "out", &vOut));
    ROCM_CALL(unwrap(inv_rms, "inv_rms", &vInv));
    ROCM_CALL(unwrap(input, "input", &vIn));
    ROCM_CALL(unwrap(weight, "weight", &vW));
    ROCM_CALL(requireDeviceContiguous(vOut, "out"));
    ROCM_CALL(requireDeviceContiguous(vInv, "inv_rms"));
    ROCM_CALL(requireDeviceContiguous(vIn, "input"));
    ROCM_CALL(requireDeviceContiguous(vW, "weight"));
    if (bias != nullptr) {
        ROCM_CALL(unwrap(bias, "bias", &vB));
        ROCM_CALL(requireDeviceContiguous(vB, "bias"));
    }
    NormDims d;
    ROCM_CALL(normDims(vIn, normalized_shape, &d));
    ROCM_CHECK(vOut.sameShape(vIn), "out must have the shape of input");
    ROCM_CHECK(isFloatDtype(vIn.dtype) && isFloatDtype(vOut.dtype), "input/out dtypes %s/%s are not supported", dtypeName(vIn.dtype),
               dtypeName(vOut.dtype));
    ROCM_CALL(checkParam(vW, "weight", normalized_shape, vOut.dtype));
    if (bias != nullptr) ROCM_CALL(checkParam(vB, "bias", normalized_shape, vOut.dtype));
    ROCM_CALL(checkInvRms(vInv, vIn, d));
    if (vIn.numel == 0) return diopiSuccess;

    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    const void* pb = bias ? vB.data : nullptr;
    // accepted (input, out) dtype pairs: layer_norm_cuda_kernel.cu:841-908 of the reference
    const diopiDtype_t ti = vIn.dtype, to = vOut.dtype;
    if (ti == diopi_dtype_float32 && to == diopi_dtype_float32) return forwardTyped<float, float>(stream, vOut, vInv, vIn, vW, pb, d, eps);
    if (ti == diopi_dtype_float16 && to == diopi_dtype_float16) return forwardTyped<half_t, half_t>(stream, vOut, vInv, vIn, vW, pb, d, eps);
    if (ti == diopi_dtype_bfloat16 && to == diopi_dtype_bfloat16) return forwardTyped<bf16_t, bf16_t>(stream, vOut, vInv, vIn, vW, pb, d, eps);
    if (ti == diopi_dtype_float32 && to == diopi_dtype_float16) return forwardTyped<float, half_t>(stream, vOut, vInv, vIn, vW, pb, d, eps);
    if (ti == diopi_dtype_float32 && to == diopi_dtype_bfloat16) return forwardTyped<float, bf16_t>(stream, vOut, vInv, vIn, vW, pb, d, eps);
    if (ti == diopi_dtype_float64 && to == diopi_dtype_float64) return forwardTyped<double, double>(stream, vOut, vInv, vIn, vW, pb, d, eps);
    if (ti == diopi_dtype_float64 && to == diopi_dtype_float32) return forwardTyped<double, float>(stream, vOut, vInv, vIn, vW, pb, d, eps);
    if (ti == diopi_dtype_float64 && to == diopi_dtype_float16) return forwardTyped<double, half_t>(stream, vOut, vInv, vIn, vW, pb, d, eps);
    if (ti == diopi_dtype_float64 && to == diopi_dtype_bfloat16) return forwardTyped<double, bf16_t>(stream, vOut, vInv, vIn, vW, pb, d, eps);
    setLastError("diopiRMSNorm: input dtype %s with out dtype %s is not supported", dtypeName(ti), dtypeName(to));
    return diopiDtypeNotSupported;
    ROCM_ENTRY_END
}

extern "C" diopiError_t diopiRMSNormBackward(diopiContextHandle_t ctx, diopiTensorHandle_t grad_input, diopiTensorHandle_t grad_weight,
                                             diopiTensorHandle_t grad_bias, diopiConstTensorHandle_t grad_output, diopiConstTensorHandle_t input,
                                             diopiConstTensorHandle_t weight, diopiConstTensorHandle_t bias, diopiConstTensorHandle_t inv_rms,
                                             diopiSize_t normalized_shape, double eps) {
    ROCM_ENTRY_BEGIN
    using namespace rocm;
    (void)bias;  // the reference ignores both (functions_ext.cpp:82-107)
    (void)eps;
    TensorView vGI, vGW, vGB, vDo, vIn, vW, vInv;
    ROCM_CALL(unwrap(grad_input, "grad_input", &vGI));
    ROCM_CALL(unwrap(grad_weight, "grad_weight", &vGW));
    ROCM_CALL(unwrap(grad_output, "grad_output", &vDo));
    ROCM_CALL(unwrap(input, "input", &vIn));
    ROCM_CALL(unwrap(weight, "weight", &vW));
    ROCM_CALL(unwrap(inv_rms, "inv_rms", &vInv));
    ROCM_CALL(requireDeviceContiguous(vGI, "grad_input"));
    ROCM_CALL(requireDeviceContiguous(vGW, "grad_weight"));
    ROCM_CALL(requireDeviceContiguous(vDo, "grad_output"));
    ROCM_CALL(requireDeviceContiguous(vIn, "input"));
    ROCM_CALL(requireDeviceContiguous(vW, "weight"));
    ROCM_CALL(requireDeviceContiguous(vInv, "inv_rms"));
    if (grad_bias != nullptr) {
        ROCM_CALL(unwrap(grad_bias, "grad_bias", &vGB));
        ROCM_CALL(requireDeviceContiguous(vGB, "grad_bias"));
    }
    NormDims d;
    ROCM_CALL(normDims(vIn, normalized_shape, &d));
    ROCM_CHECK(vGI.sameShape(vIn) && vGI.dtype == vIn.dtype, "grad_input must have the shape and dtype of input");
    ROCM_CHECK(vDo.sameShape(vIn), "grad_output must have the shape of input");
    ROCM_CHECK(isFloatDtype(vIn.dtype) && isFloatDtype(vW.dtype), "input/weight dtypes %s/%s are not supported", dtypeName(vIn.dtype),
               dtypeName(vW.dtype));
    ROCM_CALL(checkParam(vW, "weight", normalized_shape, vW.dtype));
    ROCM_CHECK(vDo.dtype == vW.dtype, "grad_output must have the dtype of weight (%s), got %s", dtypeName(vW.dtype), dtypeName(vDo.dtype));
    ROCM_CALL(checkParam(vGW, "grad_weight", normalized_shape, vW.dtype));
    if (grad_bias != nullptr) ROCM_CALL(checkParam(vGB, "grad_bias", normalized_shape, vW.dtype));
    ROCM_CALL(checkInvRms(vInv, vIn, d));
    if (d.n2 == 0) return diopiSuccess;

    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    void* pgb = grad_bias ? vGB.data : nullptr;
    if (d.n1 == 0) {
        // no rows: the column sums are empty sums
        ROCM_CALL(zeroFill(stream, vGW.data, vGW.nbytes()));
        if (pgb) ROCM_CALL(zeroFill(stream, pgb, vGB.nbytes()));
        return diopiSuccess;
    }
    const diopiDtype_t tx = vIn.dtype, tv = vW.dtype;
    if (tx == diopi_dtype_float32 && tv == diopi_dtype_float32) return backwardTyped<float, float>(ctx, stream, vGI, vGW, pgb, vDo, vIn, vW, vInv, d);
    if (tx == diopi_dtype_float16 && tv == diopi_dtype_float16) return backwardTyped<half_t, half_t>(ctx, stream, vGI, vGW, pgb, vDo, vIn, vW, vInv, d);
    if (tx == diopi_dtype_bfloat16 && tv == diopi_dtype_bfloat16)
        return backwardTyped<bf16_t, bf16_t>(ctx, stream, vGI, vGW, pgb, vDo, vIn, vW, vInv, d);
    if (tx == diopi_dtype_float32 && tv == diopi_dtype_float16) return backwardTyped<float, half_t>(ctx, stream, vGI, vGW, pgb, vDo, vIn, vW, vInv, d);
    if (tx == diopi_dtype_float32 && tv == diopi_dtype_bfloat16) return backwardTyped<float, bf16_t>(ctx, stream, vGI, vGW, pgb, vDo, vIn, vW, vInv, d);
    if (tx == diopi_dtype_float64 && tv == diopi_dtype_float64) return backwardTyped<double, double>(ctx, stream, vGI, vGW, pgb, vDo, vIn, vW, vInv, d);
    setLastError("diopiRMSNormBackward: input dtype %s with weight dtype %s is not supported", dtypeName(tx), dtypeName(tv));
    return diopiDtypeNotSupported;
    ROCM_ENTRY_END
}
