// diopiContextAttentionInference for gfx950: causal softmax(q k^T / sqrt(D)) v over packed
// variable-length sequences.
//
// Semantics: impl/torch/functions/functions_lightllm.cpp:109-147 of the reference (Python statement
// customized_test.py:8-33, 735-749).  Sequence i owns rows [b_start_loc[i], b_start_loc[i] + b_seq_len[i])
// of q, k, v and out ([rows, H, D]); inside a sequence, query row r attends to key rows 0..r.  The
// reference materialises an L x L score matrix per head, rounds it to the element type, applies an
// fp32 softmax and rounds the probabilities to the element type before the product with V.  This
// kernel keeps the fp32 scores in registers (online softmax, O(L) memory) and rounds only the
// probabilities, which stays inside the reference's 16-bit tolerance.  Rows outside every sequence
// are not written; max_input_len is not needed (the reference never reads it either).
//
// MFMA kernel (fp16 / bf16, D == 128).  A work-group of 4 or 8 waves owns 128 or 256 query rows of one
// (sequence, head); each wave owns 32 of them.  Key/value tiles of 64 rows are fetched into LDS by 16-byte buffer
// loads that write LDS directly (two buffers, one barrier per tile, a tile is requested a whole iteration before it is
// needed; packets XOR-swizzled by row so that every operand read is free of bank conflicts) and shared by the waves.
// Everything is computed transposed so that no cross-lane data movement is needed between the two matrix products:
//   S^T[key, q]  = K[key, :] . Q[q, :]      v_mfma_f32_32x32x16, A = K rows from LDS, B = Q rows (registers)
//   O^T[d, q]   += V^T[d, key] . P^T[key, q]                    A = V^T gathered from the row-major V tile, B = P^T
// In the 32x32 accumulator layout a lane holds one query column, so the row maximum, the row sum and the rescaling
// of O^T are per-lane scalars (one exchange with lane ^ 32 per tile), and the exponentiated scores are already in
// the B-operand layout of the second product.  The V^T operand comes from transposing LDS reads (ds_read_b64_tr_b16),
// two per matrix instruction.  The first product starts from the negative reference maximum and, where the scale is
// folded into the query fragments, delivers the argument of the exponential directly.
// The softmax reference maximum is updated lazily (only when it lags by more than 2^8), which keeps the rescaling
// of the 64 accumulator registers out of the common path.
// Work-groups are numbered so that the query tiles of one head land on the same XCD (they share that head's K/V
// through its L2); a small planning kernel orders the tiles of a head longest first.
//
// The same kernels serve diopiFlashAttentionVarLen (proto/include/diopi/functions_ext.h:355-359; Python statement
// customized_test.py:525-588 with multi_head_attention_inside, 36-57): sequences given by cumulative lengths, G query
// heads per key/value head, an explicit softmax scale, causal or full attention, and the row-wise log-sum-exp as a
// second output.  That form is a template flag (GEN): the lightllm operator keeps its literal scale and its
// compile-time causal structure.
#include <cmath>
#include <cstdlib>
#include <mutex>
#include <type_traits>

#include "common.hpp"
#include "device.hpp"

namespace rocm {
namespace {

constexpr int kBMMin = 128;  // smallest query tile of a work-group (bounds of the planning step are sized for it)
constexpr int kBN = 64;    // key rows per tile
constexpr int kHD = 128;   // head size of the MFMA kernel
constexpr int kLD = kHD + 8;  // row pitch of the output tile in LDS, in elements (272 bytes: 16-byte aligned)
typedef short s16x4 __attribute__((ext_vector_type(4)));
constexpr float kLazyLog2 = 8.0f;  // how far (in powers of two) the softmax reference maximum may lag behind
// The same for the pipelined kernel's main loop, which pays for a move of the reference with the rest of the wave's tiles at
// the plain loop's speed: probabilities up to 2^14 still fit the 16-bit types with full relative precision.
constexpr float kPipeLazyLog2 = 14.0f;

struct CtxArgs {
    const void* bStartLoc;
    const void* bSeqLen;
    bool start64, len64;
    int batch;
    int H;
    int64_t rows;      // rows of q / k / v / out
    const int4* plan;  // [tilesBound] visiting order of the query tiles of one head, written by ctxAttnPlan
    int tilesBound;    // upper bound on the number of 128-row query tiles over all sequences
    int totalItems;    // H * tilesBound
    // general form only (diopiFlashAttentionVarLen); the lightllm operator leaves these at their defaults
    bool cumulative;   // bStartLoc holds batch + 1 cumulative lengths; bSeqLen is unused
    int uniformLen;    // > 0: every sequence has this many rows and sequence i starts at row i * uniformLen (no index tensors)
    bool causal;
    int G;             // query heads per key/value head
    float scaleLog2;   // softmax scale * log2(e)
    float* lse;        // [batch, H, lseStride] log-sum-exp of the scaled scores of every query row, or null
    int lseStride;     // max_seqlen_q
};

// Where a call keeps its tile plan: in scratch of the caller's context (the default), or in the library's own static
// device array (the allocation-free entry point).
struct PlanStore {
    int4* fixed = nullptr;  // device address of the static array on the current device, or null: ask the context
    int capacity = 0;       // entries of the static array
};

// Tile plans of the allocation-free entry point.  One array per device the library runs on, held until the process
// ends; every call on a device shares it, so such calls must not overlap on one device.
constexpr int kStaticPlanEntries = 8192;  // 128 KiB: query tiles + sequences of one call
static __device__ __align__(256) int4 scratch[kStaticPlanEntries];

template <typename T>
struct Mfma32;
template <>
struct Mfma32<half_t> {
    using Frag = f16x8;
    static __device__ __forceinline__ f32x16 mma(Frag a, Frag b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
    // acc + lo + hi of a packed pair, in one instruction
    static __device__ __forceinline__ float addPair(uint32_t pair, float acc) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        const h2 ones = {static_cast<_Float16>(1.f), static_cast<_Float16>(1.f)};
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, pair), ones, acc, false);
    }
};
template <>
struct Mfma32<bf16_t> {
    using Frag = bf16x8;
    static __device__ __forceinline__ f32x16 mma(Frag a, Frag b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ float addPair(uint32_t pair, float acc) {
        typedef __bf16 b2 __attribute__((ext_vector_type(2)));
        const b2 ones = {static_cast<__bf16>(1.f), static_cast<__bf16>(1.f)};
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b2, pair), ones, acc, false);
    }
};

template <typename Frag>
union FragBits {
    u32x4 raw;
    Frag f;
    __device__ FragBits() {}
};

// One 16-byte load per lane from a raw buffer straight into LDS: lane l's packet lands at ldsAddr + 16 l.  The LDS
// base travels in M0 (wave-uniform).  Written as assembly so that the compiler does not order later LDS reads of
// other addresses behind the load; the issuer must call waitLdsLoads() before the barrier that publishes the data.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void loadToLds16(u32x4 rsrc, uint32_t ldsAddr, int byteOffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(ldsAddr), "v"(byteOffset), "s"(rsrc) : "memory", "m0");
}
#pragma clang diagnostic pop
__device__ __forceinline__ void waitLdsLoads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// max(v, v of lane ^ 32) without a trip through the LDS crossbar: v_permlane32_swap exchanges the upper half of its
// first operand with the lower half of its second, so two copies of v become (lower half twice, upper half twice).
// The instruction is written out because the compiler's builtin returns the first result twice; the s_nop cover the
// wait states the instruction needs next to vector instructions that write or read its operands.
__device__ __forceinline__ float maxWithOtherHalf(float v) {
    float lo = v, hi = v;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
    return fmaxf(lo, hi);
}

// max(a, b, c) as the one instruction it is.  Written out because fmaxf on values the compiler cannot prove to be
// quiet numbers first canonicalises each of them (a v_max_f32 x, x, x apiece: 12 extra vector instructions per key tile);
// the scores are sums of finite products or the mask's -1e30, never signalling NaNs.
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// Sequence geometry with every value forced inside the tensors.
struct SeqInfo {
    int64_t start;
    int64_t len;
};

__device__ __forceinline__ SeqInfo loadSeq(const CtxArgs& a, int i) {
    SeqInfo s;
    if (a.uniformLen > 0) {
        s.start = static_cast<int64_t>(i) * a.uniformLen;
        s.len = a.uniformLen;
        return s;
    }
    s.start = loadIndex(a.bStartLoc, i, a.start64);
    s.len = a.cumulative ? loadIndex(a.bStartLoc, i + 1, a.start64) - s.start : loadIndex(a.bSeqLen, i, a.len64);
    if (s.start < 0 || s.start >= a.rows) s.len = 0;
    if (s.len > a.rows - s.start) s.len = a.rows - s.start;
    if (s.len < 0) s.len = 0;
    return s;
}

// Visiting order of the query tiles of one head: entry p of `plan` is (sequence, query tile index, first row and
// length of the sequence: everything a work-group needs, in one load), sorted by tile
// index descending.  A query tile with index t attends to t + 1 key blocks, so this is longest-job-first and the
// short tiles fill the tail of the launch whatever the mix of sequence lengths.  With the sequences ranked by tile
// count (descending), the sequences that own a tile of index t are a prefix of that ranking, hence
//   position(seq, t) = sum_s max(0, tiles_s - 1 - t)  +  rank(seq).
// One work-group; tile counts are kept in LDS.  Unused entries (the bound over-counts) get sequence -1.
constexpr int kPlanThreads = 1024;
__global__ __launch_bounds__(kPlanThreads) void ctxAttnPlan(int4* __restrict__ plan, CtxArgs a, int maxTiles, int bm) {
    extern __shared__ int sTiles[];  // [batch] tile counts, [batch] ranks, [maxTiles] offsets, [2 * batch] geometry
    const int tid = threadIdx.x;
    int* sStart = sTiles + 2 * a.batch + maxTiles;  // [batch] first row, then [batch] length (the launcher checked that row counts fit 32 bits)
    for (int s = tid; s < a.batch; s += kPlanThreads) {
        const SeqInfo si = loadSeq(a, s);
        sTiles[s] = static_cast<int>((si.len + bm - 1) / bm);
        sStart[s] = static_cast<int>(si.start);
        sStart[a.batch + s] = static_cast<int>(si.len);
    }
    for (int p = tid; p < a.tilesBound; p += kPlanThreads) plan[p] = make_int4(-1, 0, 0, 0);
    __syncthreads();
    for (int s = tid; s < a.batch; s += kPlanThreads) {
        const int nt = sTiles[s];
        if (nt == 0) continue;
        int rank = 0;
        for (int s2 = 0; s2 < a.batch; ++s2) {
            const int nt2 = sTiles[s2];
            rank += (nt2 > nt || (nt2 == nt && s2 < s)) ? 1 : 0;
        }
        sTiles[a.batch + s] = rank;
    }
    __syncthreads();
    for (int t = tid; t < maxTiles; t += kPlanThreads) {
        int off = 0;
        for (int s = 0; s < a.batch; ++s) {
            const int more = sTiles[s] - 1 - t;
            off += more > 0 ? more : 0;
        }
        sTiles[2 * a.batch + t] = off;
    }
    __syncthreads();
    for (int s = 0; s < a.batch; ++s) {
        const int nt = sTiles[s];
        const int rank = nt > 0 ? sTiles[a.batch + s] : 0;
        for (int t = tid; t < nt; t += kPlanThreads) {
            // overlapping sequences (a caller error) could count more tiles than the bound the table is sized for
            const int pos = (t < maxTiles ? sTiles[2 * a.batch + t] : a.tilesBound) + rank;
            if (pos < a.tilesBound) plan[pos] = make_int4(s, t, sStart[s], sStart[a.batch + s]);
        }
    }
}

template <typename T, int NWV, bool GEN>
__global__ __launch_bounds__(NWV * kWave, NWV == 4 ? 2 : 1) void ctxAttnMfma(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                                                               CtxArgs a) {
    // exp(x / sqrt(D)) = exp2(x * log2(e) / sqrt(D)): one literal factor (a run-time one in the general form)
    constexpr float kScaleLog2 = 0.12751743082459868f;  // log2(e) / sqrt(128)
    const float scaleLog2 = GEN ? a.scaleLog2 : kScaleLog2;
    const bool causal = GEN ? a.causal : true;
    using Ops = Mfma32<T>;
    using Frag = typename Ops::Frag;
    constexpr int BM = NWV * 32;  // query rows per work-group: each of the NWV waves owns 32 of them
    // two staging buffers of (K tile, V tile), both [key][dim] row-major with swizzled 16-byte packets, see below
    extern __shared__ __attribute__((aligned(16))) unsigned char dynSmem[];
    T* smem = reinterpret_cast<T*>(dynSmem);

    // ---- which (head, sequence, query tile) is this work-group? ----
    const int perXcd = (a.totalItems + kNumXcd - 1) / kNumXcd;
    const int item = (blockIdx.x % kNumXcd) * perXcd + blockIdx.x / kNumXcd;
    if (item >= a.totalItems) return;
    const int head = item / a.tilesBound;
    const int tileFlat = item % a.tilesBound;
    const int4 planned = a.plan[tileFlat];  // (sequence, query tile, first row, length), longest tiles first; sequence -1 = padding
    if (planned.x < 0) return;
    const int qt = planned.y;
    SeqInfo si;
    si.start = planned.z;
    si.len = planned.w;
    const int L = static_cast<int>(si.len);              // the launcher checked that row counts fit 32 bits
    const int m0 = qt * BM;

    const int tid = threadIdx.x;
    const int lane = tid % kWave;
    const int wave = tid / kWave;
    const int n = lane % 32;   // query column of this lane in every accumulator
    const int hh = lane / 32;  // which half of the k slots / which 4-row sub-block of the accumulator
    const int64_t qPitch = static_cast<int64_t>(a.H) * kHD;                   // row pitch of q and out
    const int64_t rowPitch = GEN ? static_cast<int64_t>(a.H / a.G) * kHD : qPitch;  // row pitch of k and v
    const int kvHead = GEN ? head / a.G : head;
    const T* qBase = q + si.start * qPitch + static_cast<int64_t>(head) * kHD;
    const T* kBase = k + si.start * rowPitch + static_cast<int64_t>(kvHead) * kHD;
    const T* vBase = v + si.start * rowPitch + static_cast<int64_t>(kvHead) * kHD;

    // ---- Q fragments (B operand of S^T): row = m0 + 32*wave + n, k slot (hh, e) <-> dim 16*s + 8*hh + e ----
    // The query is multiplied by softmax_scale * log2(e) here, once, so that the first product delivers the exponent
    // of 2 directly.  That rounds the scaled query to the element type, the size of the rounding the reference applies
    // to its scores (functions_lightllm.cpp:121 keeps them in the tensor dtype).  The general form with bf16 tensors
    // (8 bits) does not: it also returns the log-sum-exp, which would inherit that rounding; it keeps the
    // multiplication in fp32, one instruction per score, and sums the unrounded probabilities.
    constexpr bool kFold = std::is_same<T, half_t>::value || !GEN;
    const float toLog2 = kFold ? 1.f : scaleLog2;  // from the unit of the score accumulators to powers of two
    const int qRow = m0 + wave * 32 + n;
    const int qRowLd = qRow < L ? qRow : L - 1;
    Frag qf[kHD / 16];
#pragma unroll
    for (int s = 0; s < kHD / 16; ++s) {
        FragBits<Frag> u;
        u.raw = *reinterpret_cast<const u32x4*>(qBase + qRowLd * qPitch + s * 16 + hh * 8);
        if constexpr (kFold) {
#pragma unroll
            for (int e = 0; e < 8; ++e) qf[s][e] = static_cast<T>(static_cast<float>(u.f[e]) * scaleLog2);
        } else {
            qf[s] = u.f;
        }
    }

    f32x16 o[kHD / 32];
#pragma unroll
    for (int mb = 0; mb < kHD / 32; ++mb) {
#pragma unroll
        for (int r = 0; r < 16; ++r) o[mb][r] = 0.f;
    }
    // Reference maximum of this lane's query row in the unit of the score accumulators, and its negative in all 16
    // registers of an accumulator tuple: the first product of a tile starts from it, so the scores arrive as
    // (score - reference), ready for the exponential.
    float mRun = 0.f;
    f32x16 negRef;
#pragma unroll
    for (int r = 0; r < 16; ++r) negRef[r] = 0.f;
    float lRun = 0.f;  // this lane's share of the row sum (the other half lives in lane ^ 32)

    const int kEnd = (causal && m0 + BM < L) ? m0 + BM : L;  // keys 0 .. kEnd-1 are visible to this tile
    const int numKeyTiles = (kEnd + kBN - 1) / kBN;
    const int waveRowLo = m0 + wave * 32;
    const int waveRowHi = waveRowLo + 31;

    // ---- tile staging: 16-byte loads that land in LDS directly (no registers, no LDS write instructions) ----
    // One such load of a wave fills 1 KB of consecutive LDS (lane l writes bytes 16 l .. 16 l + 15), i.e. 4 rows of
    // a [64 keys][256 bytes] tile; which 16-byte packet of its row a lane fetches is free, and that is where the
    // bank-conflict avoidance goes, since the rows cannot be padded:
    //   K tile: slot s of row r holds packet s ^ (r & 15)      (16 lanes reading one packet of 16 rows hit 16 slots)
    //   V tile: slot s of row r holds packet s ^ (4 * (r & 3)) (see the transposing reads below)
    // Rows past the sequence are outside the tile's buffer descriptor and arrive as zeros; they are masked below.
    constexpr int kTileBytes = kBN * kHD * static_cast<int>(sizeof(T));  // 16 KB
    constexpr int kBufBytes = 2 * kTileBytes;                          // K tile, then V tile
    constexpr int kChunks = kBN / 4 / NWV;                             // 1 KB pieces per wave and tile: 4 or 2
    using LdsByte = __attribute__((address_space(3))) unsigned char;
    LdsByte* const lds = (LdsByte*)dynSmem;
    const uint32_t ldsBase = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));
    const int waveU = __builtin_amdgcn_readfirstlane(wave);
    const int rowBytes = static_cast<int>(rowPitch) * static_cast<int>(sizeof(T));  // the launcher bounds 64 rows by 2^31 bytes
    int kSrc[kChunks], vSrc[kChunks];
#pragma unroll
    for (int it = 0; it < kChunks; ++it) {
        const int r = (waveU * kChunks + it) * 4 + lane / 16;
        kSrc[it] = r * rowBytes + (((lane % 16) ^ (r & 15)) * 16);
        vSrc[it] = r * rowBytes + (((lane % 16) ^ (4 * (r & 3))) * 16);
    }
    // Requests the next tile into the buffer the previous one left.  The scalar state (tile addresses, LDS address)
    // advances from call to call so that a request costs a handful of scalar instructions; the last tile of a
    // sequence gets a shorter descriptor (rows past the sequence read as zeros), tiles past the last are not requested.
    const int64_t tileBytes = static_cast<int64_t>(kBN) * rowPitch * static_cast<int64_t>(sizeof(T));
    const int fullBytes = static_cast<int>(((kBN - 1) * rowPitch + kHD) * static_cast<int64_t>(sizeof(T)));
    const int lastBytes = static_cast<int>(((L - (numKeyTiles - 1) * kBN - 1) * rowPitch + kHD) * static_cast<int64_t>(sizeof(T)));
    uint64_t kNext = reinterpret_cast<uint64_t>(kBase);
    uint64_t vNext = reinterpret_cast<uint64_t>(vBase);
    uint32_t dstNext = ldsBase + waveU * kChunks * 1024;
    int nextTile = 0;
    auto requestNext = [&]() {
        if (nextTile < numKeyTiles) {  // wave-uniform
            const uint32_t bytes = static_cast<uint32_t>(nextTile == numKeyTiles - 1 && L < numKeyTiles * kBN ? lastBytes : fullBytes);
            const u32x4 kBuf = {static_cast<uint32_t>(kNext), static_cast<uint32_t>(kNext >> 32) & 0xffffu, bytes, kRawBufferWord3};
            const u32x4 vBuf = {static_cast<uint32_t>(vNext), static_cast<uint32_t>(vNext >> 32) & 0xffffu, bytes, kRawBufferWord3};
#pragma unroll
            for (int it = 0; it < kChunks; ++it) {
                loadToLds16(kBuf, dstNext + it * 1024, kSrc[it]);
                loadToLds16(vBuf, dstNext + kTileBytes + it * 1024, vSrc[it]);
            }
        }
        kNext += tileBytes;
        vNext += tileBytes;
        dstNext ^= kBufBytes;
        ++nextTile;
    };
    requestNext();
    // ---- operand addresses inside a buffer ----
    // K (A operand of S^T): row 32 sb + n, packet 2 st + hh, one 16-byte read.
    // V^T (A operand of O^T): a lane needs 8 keys of one dim, which in the row-major V tile are 8 rows apart by 256
    // bytes.  The transposing read ds_read_b64_tr_b16 does the gather: inside a group of 16 lanes, lane (kk, q)
    // (= lane % 16 / 4, lane % 4) supplies the address of 4 consecutive dims of key kk, and lane i receives element
    // i % 4 of the 4 addresses given by lanes i / 4, i / 4 + 4, i / 4 + 8, i / 4 + 12: keys 0..3 of dim 4 (i / 4) + i % 4.
    // Lane group g16 = lane / 16 covers dims 16 (g16 % 2) .. + 15 of a 32-dim block and keys 4 hh .. + 3 of an 8-key
    // half; two reads (halves 0 and 1) give the 8 k slots of a lane in the order in which the first product leaves
    // the probabilities (k slot (hh, j) of a 16-key group is key 8 (j / 4) + 4 hh + j % 4).  The 4 * (r & 3) swizzle
    // spreads the 4 keys x 4 packets that 32 lanes touch at once over 16 different slots.
    int kOff[kHD / 16], vOff[kHD / 32];
    {
        const int hx = hh ^ (n & 15);
#pragma unroll
        for (int st = 0; st < kHD / 16; ++st) kOff[st] = n * 256 + (((2 * st) ^ hx) * 16);
        const int g16 = lane / 16, kk = (lane % 16) / 4, qq = lane % 4;
        const int cLo = 2 * (g16 % 2) + qq / 2;
#pragma unroll
        for (int mb = 0; mb < kHD / 32; ++mb) vOff[mb] = kTileBytes + (4 * hh + kk) * 256 + ((4 * (mb ^ kk) + cLo) * 16) + (qq % 2) * 8;
    }

    // The query fragments must have arrived before the loop: a wait for them inside it would also wait for the tile
    // requests, which the compiler does not count.
#pragma unroll
    for (int s = 0; s < kHD / 16; ++s) asm volatile("" : "+v"(qf[s]));

    for (int jt = 0; jt < numKeyTiles; ++jt) {
        // One barrier per tile: tile jt has landed (every wave waits for its own requests before the barrier) and
        // every wave has left tile jt-1, whose buffer the request for tile jt+1 now fills while this tile is used.
        waitLdsLoads();
        __syncthreads();
        const LdsByte* sBuf = lds + (jt & 1) * kBufBytes;
        const int key0 = jt * kBN;
        // nothing to do for this wave: the tile lies entirely above the diagonal, or the wave's 32 rows lie past the
        // sequence (the last query tile of a sequence is rarely full; such a wave only fetches its share of the tiles)
        const bool skip = (causal && key0 > waveRowHi) || waveRowLo >= L;

        // ---- S^T = K . Q^T for the two 32-key blocks ----
        // LDS operands are requested one step ahead of the product that consumes them, and the two key blocks
        // alternate so that consecutive products never wait on each other's accumulator.  The first operands are
        // requested before the scalar work of the tile request, which then runs while they travel.
        constexpr int kKDepth = 2;  // K operand steps in flight: LDS latency under load spans several products
        FragBits<Frag> kf[kKDepth][2];
        auto loadK = [&](int st, int b) {
#pragma unroll
            for (int sb = 0; sb < 2; ++sb) kf[b][sb].raw = *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(sBuf + kOff[st] + sb * 32 * 256);
        };
        if (!skip) {
#pragma unroll
            for (int st = 0; st < kKDepth - 1; ++st) loadK(st, st);
        }
        requestNext();
        if (skip) continue;  // barriers are at the loop top
        f32x16 s[2];
        s[0] = negRef;
        s[1] = negRef;
#pragma unroll
        for (int st = 0; st < kHD / 16; ++st) {
            if (st + kKDepth - 1 < kHD / 16) loadK(st + kKDepth - 1, (st + kKDepth - 1) % kKDepth);
            __builtin_amdgcn_sched_barrier(0);  // keep the read-ahead order: the scheduler would otherwise sink the reads
            s[0] = Ops::mma(kf[st % kKDepth][0].f, qf[st], s[0]);
            s[1] = Ops::mma(kf[st % kKDepth][1].f, qf[st], s[1]);
            __builtin_amdgcn_sched_barrier(0);
        }
        // V^T operands of the first 16-key group travel while the softmax runs
        FragBits<Frag> vf[2][kHD / 32];
        auto loadV = [&](int g, int b) {
#pragma unroll
            for (int mb = 0; mb < kHD / 32; ++mb) {
#pragma unroll
                for (int h2 = 0; h2 < 2; ++h2) {
                    using Quad = __attribute__((address_space(3))) s16x4;
                    const s16x4 t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((Quad*)(sBuf + vOff[mb] + (16 * g + 8 * h2) * 256));
                    vf[b][mb].raw[2 * h2] = __builtin_bit_cast(u32x2, t)[0];
                    vf[b][mb].raw[2 * h2 + 1] = __builtin_bit_cast(u32x2, t)[1];
                }
            }
        };
        loadV(0, 0);
        __builtin_amdgcn_sched_barrier(0);
        // accumulator register r of block sb holds key  key0 + 32*sb + 8*(r/4) + 4*hh + r%4  for query row qRow
        if (causal ? key0 + kBN - 1 > waveRowLo : key0 + kBN > L) {
            // causal: keys past the query's own position (which covers keys past the sequence, which arrive as
            // zeros); full attention: only those
            const int lastKey = causal ? qRow : L - 1;
#pragma unroll
            for (int sb = 0; sb < 2; ++sb) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = key0 + sb * 32 + (r / 4) * 8 + hh * 4 + (r % 4);
                    if (key > lastKey) s[sb][r] = -1e30f;
                }
            }
        }
        // largest score of the tile relative to the reference: four independent chains, then the other lane half
        float tm[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int sb = c / 2, r0 = 8 * (c % 2);
            tm[c] = max3(s[sb][r0], s[sb][r0 + 1], s[sb][r0 + 2]);
            tm[c] = max3(tm[c], s[sb][r0 + 3], s[sb][r0 + 4]);
            tm[c] = max3(tm[c], s[sb][r0 + 5], s[sb][r0 + 6]);
        }
        const float tmA = max3(tm[0], s[0][7], s[0][15]), tmB = max3(tm[1], s[1][7], s[1][15]);
        float tmLo = max3(max3(tmA, tmB, tm[2]), tm[3], tm[3]);  // this lane's 32 scores
        float tmHi = tmLo;
        asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(tmLo), "+v"(tmHi));  // see maxWithOtherHalf
        const float tmax = max3(tmLo, tmHi, tmHi);
        // The reference only follows the true maximum when it has fallen behind by more than 2^kLazyLog2 (a
        // wave-uniform, rarely taken branch after the first tile, where it is set for the first time): probabilities
        // then reach at most 2^kLazyLog2, which the 16-bit types hold with full relative precision, and the
        // accumulators are rescaled only then.
        if (jt == 0 || __any(tmax * toLog2 > kLazyLog2)) {
            const float up = jt == 0 ? tmax : fmaxf(tmax, 0.f);
            const float alpha = __builtin_amdgcn_exp2f(-up * toLog2);
            mRun += up;
            lRun *= alpha;
#pragma unroll
            for (int r = 0; r < 16; ++r) negRef[r] = -mRun;
#pragma unroll
            for (int mb = 0; mb < kHD / 32; ++mb) {
#pragma unroll
                for (int r = 0; r < 16; ++r) o[mb][r] *= alpha;
            }
#pragma unroll
            for (int sb = 0; sb < 2; ++sb) {
#pragma unroll
                for (int r = 0; r < 16; ++r) s[sb][r] -= up;
            }
        }
        // ---- probabilities and O^T += V^T . P^T, one group of 16 keys at a time ----
        // k slot (hh, j) of group g = 2*sb + u is key 16*g + 8*(j/4) + 4*hh + j%4; accumulator row n' of o[mb] stands
        // for dim 32*mb + n'.  The exponentials of a group are issued right before its four products, so that they run
        // while the matrix pipe works on the previous group's (of this wave and of the other wave of the SIMD).
        float psum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int sb = g / 2, u = g % 2;
            FragBits<Frag> pk;
            if constexpr (kFold) {
#pragma unroll
                for (int j = 0; j < 8; ++j) pk.f[j] = static_cast<T>(__builtin_amdgcn_exp2f(s[sb][u * 8 + j]));
                // the row sum takes the rounded probabilities (the ones the second product multiplies), two per instruction
#pragma unroll
                for (int w = 0; w < 4; ++w) psum[w] = Ops::addPair(pk.raw[w], psum[w]);
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float p = __builtin_amdgcn_exp2f(s[sb][u * 8 + j] * scaleLog2);
                    psum[j & 3] += p;
                    pk.f[j] = static_cast<T>(p);
                }
            }
            if (g + 1 < 4) loadV(g + 1, (g + 1) & 1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int mb = 0; mb < kHD / 32; ++mb) o[mb] = Ops::mma(vf[g & 1][mb].f, pk.f, o[mb]);
            __builtin_amdgcn_sched_barrier(0);
        }
        lRun += (psum[0] + psum[1]) + (psum[2] + psum[3]);
    }

    // ---- normalise, transpose through LDS, write rows with 16-byte stores ----
    const float lTot = lRun + __shfl_xor(lRun, 32, kWave);
    const float inv = 1.0f / lTot;
    if constexpr (GEN) {
        // ln sum_j exp(scale * s_j) = ln 2 * (reference maximum in log2 units + log2 of the sum relative to it)
        if (a.lse != nullptr && hh == 0 && qRow < L && qRow < a.lseStride)
            a.lse[(static_cast<int64_t>(planned.x) * a.H + head) * a.lseStride + qRow] = 0.6931471805599453f * (mRun * toLog2 + __builtin_amdgcn_logf(lTot));
    }
    waitLdsLoads();
    __syncthreads();  // the K/V tiles are dead and no request is in flight; reuse the storage as a [BM][kLD] output tile
    T* sO = smem;
    static_assert(kHD == 128, "scaleLog2 is written out for head size 128");
#pragma unroll
    for (int mb = 0; mb < kHD / 32; ++mb) {
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
            // registers 4 rq .. 4 rq + 3 of o[mb] are dims 32 mb + 8 rq + 4 hh .. + 3
            T pk[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) pk[e] = static_cast<T>(o[mb][4 * rq + e] * inv);
            *reinterpret_cast<u32x2*>(sO + (wave * 32 + n) * kLD + 32 * mb + 8 * rq + 4 * hh) = *reinterpret_cast<const u32x2*>(pk);
        }
    }
    // each wave only reads back the 32 rows it wrote: no work-group barrier needed, LDS ops of a wave are ordered
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    T* oBase = out + si.start * qPitch + static_cast<int64_t>(head) * kHD;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const int id = it * kWave + lane;
        const int row = id / 16;
        const int c = id % 16;
        const int grow = m0 + wave * 32 + row;
        if (grow < L) {
            const u32x4 val = *reinterpret_cast<const u32x4*>(sO + (wave * 32 + row) * kLD + c * 8);
            *reinterpret_cast<u32x4*>(oBase + grow * qPitch + c * 8) = val;
        }
    }
}

// v_mfma_f32_32x32x16 written out, accumulating in place.  The compiler does not see a matrix instruction in it, so it
// inserts none of the wait states a read of the result by a vector instruction needs shortly after (11 for this 8-pass
// shape); mfmaSettle() provides them where such a read follows within a few instructions.  In return the accumulators
// stay where they are: with the builtin, a path that rewrites accumulators (the rare move of the softmax reference) made
// the compiler settle the two paths' registers with a copy of every accumulator on the common path.
template <typename T>
struct MfmaInPlace;
template <>
struct MfmaInPlace<half_t> {
    static __device__ __forceinline__ void acc(f32x16& c, u32x4 a, f16x8 b) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ void start(f32x16& d, u32x4 a, f16x8 b, const f32x16& c) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(d) : "v"(a), "v"(b), "v"(c));
    }
};
template <>
struct MfmaInPlace<bf16_t> {
    static __device__ __forceinline__ void acc(f32x16& c, u32x4 a, bf16x8 b) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ void start(f32x16& d, u32x4 a, bf16x8 b, const f32x16& c) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(d) : "v"(a), "v"(b), "v"(c));
    }
};
// The wait runs through the registers it is for: a read of them that only depended on the product could be scheduled ahead of
// the wait itself (a maximum taken from a score tuple one product short moves the softmax reference too little, and a
// probability past 2^16 leaves the 16-bit range).
__device__ __forceinline__ void mfmaSettle(f32x16& a) { asm volatile("s_nop 7\n\ts_nop 3" : "+v"(a)); }
__device__ __forceinline__ void mfmaSettle(f32x16& a, f32x16& b) { asm volatile("s_nop 7\n\ts_nop 3" : "+v"(a), "+v"(b)); }
__device__ __forceinline__ void mfmaSettle(f32x16& a, f32x16& b, f32x16& c, f32x16& d) {
    asm volatile("s_nop 7\n\ts_nop 3" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}

// The lightllm prefill operator as one software-pipelined instruction stream per wave (fp16 / bf16, D == 128, causal).
//
// What the hardware does (measured): a matrix instruction keeps the SIMD's vector issue port for about 8 clocks whatever
// its shape, and one that waits for the matrix pipe holds the port until it is issued.  Two waves that alternate between
// blocks of products and blocks of vector work therefore do not overlap them, the blocks add up; and the 16x16x32 shape,
// with twice the instructions per flop, leaves too little of the port for the softmax.  So: v_mfma_f32_32x32x16 (32
// clocks of pipe, about 24 of them free for vector instructions), and every product is followed at once by its share of
// the vector work of ANOTHER half tile, a few instructions that depend on nothing recent, so that the next product
// arrives about when the pipe frees.  A key tile of 64 rows is handled as two halves of 32 keys; with (jt, h) the half h
// of tile jt, one trip of the loop is
//   phase 1:  S^T(jt, 1) = K . Q^T        8 products, between them the 16 exponentials and 8 packed conversions of (jt, 0)
//   phase 2:  O^T += V^T(jt, 0) . P^T      8 products, between them the row sums of (jt, 0) and the maximum of (jt, 1)
//   phase 3:  S^T(jt + 1, 0)               ... and the exponentials of (jt, 1)
//   phase 4:  O^T += V^T(jt, 1) . P^T      ... and the row sums of (jt, 1), the maximum of (jt + 1, 0)
// The K tile runs half a tile ahead of the V tile in LDS (two buffers each).  The last tile of a wave, the one its
// diagonal crosses, is masked and finished outside the pipeline, and so is everything after a move of the softmax
// reference (rare: see kPipeLazyLog2).  Layouts as in ctxAttnMfma: a lane owns query row lane % 32.
template <typename T, int NWV>
__global__ __launch_bounds__(NWV * kWave, NWV == 4 ? 2 : 1) void ctxAttnPipe(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k,
                                                                               const T* __restrict__ v, CtxArgs a) {
    constexpr float kScaleLog2 = 0.12751743082459868f;  // log2(e) / sqrt(128)
    using Ops = MfmaInPlace<T>;
    using Sum = Mfma32<T>;
    using Frag = typename Mfma32<T>::Frag;
    constexpr int BM = NWV * 32;
    constexpr int kKRing = 3, kVRing = 3;  // operand fragments in registers: read-ahead = ring - 1 products
    extern __shared__ __attribute__((aligned(16))) unsigned char dynSmem[];
    T* smem = reinterpret_cast<T*>(dynSmem);

    const int perXcd = (a.totalItems + kNumXcd - 1) / kNumXcd;
    const int item = (blockIdx.x % kNumXcd) * perXcd + blockIdx.x / kNumXcd;
    if (item >= a.totalItems) return;
    const int head = item / a.tilesBound;
    const int4 planned = a.plan[item % a.tilesBound];
    if (planned.x < 0) return;
    const int qt = __builtin_amdgcn_readfirstlane(planned.y);
    const int64_t seqStart = __builtin_amdgcn_readfirstlane(planned.z);
    const int L = __builtin_amdgcn_readfirstlane(planned.w);
    const int m0 = qt * BM;

    const int tid = threadIdx.x;
    const int lane = tid % kWave;
    const int wave = tid / kWave;
    const int n = lane % 32;   // query column of this lane in every accumulator
    const int hh = lane / 32;  // which half of the k slots / which 4-row sub-block of the accumulator
    const int64_t qPitch = static_cast<int64_t>(a.H) * kHD;
    const T* qBase = q + seqStart * qPitch + static_cast<int64_t>(head) * kHD;
    const T* kBase = k + seqStart * qPitch + static_cast<int64_t>(head) * kHD;
    const T* vBase = v + seqStart * qPitch + static_cast<int64_t>(head) * kHD;

    // ---- Q^T fragments (B operand of the first product): query row n, dims 16 st + 8 hh .. + 7, scaled by
    // log2(e) / sqrt(D) and rounded to the element type once (see ctxAttnMfma) ----
    Frag qf[kHD / 16];
    {
        const int row = m0 + wave * 32 + n;
        const int rowLd = row < L ? row : L - 1;
#pragma unroll
        for (int st = 0; st < kHD / 16; ++st) {
            FragBits<Frag> u;
            u.raw = *reinterpret_cast<const u32x4*>(qBase + rowLd * qPitch + st * 16 + hh * 8);
#pragma unroll
            for (int e = 0; e < 8; ++e) qf[st][e] = static_cast<T>(static_cast<float>(u.f[e]) * kScaleLog2);
        }
    }

    f32x16 o[kHD / 32];
#pragma unroll
    for (int mb = 0; mb < kHD / 32; ++mb) {
#pragma unroll
        for (int r = 0; r < 16; ++r) o[mb][r] = 0.f;
    }
    f32x16 s0, s1;     // scores of the lower / upper 32 keys of a tile: register r is key 8 (r / 4) + 4 hh + r % 4
    float lRun = 0.f;  // this lane's share of the row sum (the other half lives in lane ^ 32)
    // minus the reference maximum of the lane's query row (in powers of two), as the accumulator the first product of a
    // half starts from: the scores arrive as score - reference, ready for the exponential
    f32x16 negRef;
#pragma unroll
    for (int r = 0; r < 16; ++r) negRef[r] = 0.f;
    Frag pf[2];        // probabilities of one half, per group of 16 keys

    const int kEnd = m0 + BM < L ? m0 + BM : L;
    const int numKeyTiles = (kEnd + kBN - 1) / kBN;

    // ---- tile staging (see ctxAttnMfma): K tile c in buffer c & 1 at 32 KiB * (c & 1), V tile c of buffer c & 1 16 KiB behind it ----
    constexpr int kTileBytes = kBN * kHD * static_cast<int>(sizeof(T));
    constexpr int kChunks = kBN / 4 / NWV;
    using LdsByte = __attribute__((address_space(3))) unsigned char;
    LdsByte* const lds = (LdsByte*)dynSmem;
    const uint32_t ldsBase = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));
    const int waveU = __builtin_amdgcn_readfirstlane(wave);
    const int waveRowLo = m0 + waveU * 32;
    const bool active = waveRowLo < L;
    const int dg = waveRowLo / kBN;  // the tile this wave's diagonal crosses, its last one
    const int rowBytes = static_cast<int>(qPitch) * static_cast<int>(sizeof(T));
    int kSrc[kChunks], vSrc[kChunks];
#pragma unroll
    for (int it = 0; it < kChunks; ++it) {
        const int r = (waveU * kChunks + it) * 4 + lane / 16;
        kSrc[it] = r * rowBytes + (((lane % 16) ^ (r & 15)) * 16);
        vSrc[it] = r * rowBytes + (((lane % 16) ^ (4 * (r & 3))) * 16);
    }
    // The K tiles are cut half a tile off the V tiles: K tile c holds key rows 64 c - 32 .. 64 c + 31, because one trip of
    // the loop multiplies by the upper half of one 64-key tile and the lower half of the next, and a buffer can only be
    // refilled once every wave has left it.  K tile 0 therefore has no lower half (nothing is fetched for it), and there
    // is one K tile more than V tiles.  Rows past the sequence are outside the tile's buffer descriptor and arrive as zeros.
    const int64_t tileStride = static_cast<int64_t>(kBN) * qPitch * static_cast<int64_t>(sizeof(T));
    // the tile addresses live in scalar registers (the sequence's first row came from memory, into a vector register)
    uint64_t kNext = reinterpret_cast<uint64_t>(uniformPointer(kBase)) - static_cast<uint64_t>(tileStride / 2);
    uint64_t vNext = reinterpret_cast<uint64_t>(uniformPointer(vBase));
    uint32_t kDst = ldsBase + waveU * kChunks * 1024, vDst = ldsBase + kTileBytes + waveU * kChunks * 1024;
    int kRow = -kBN / 2, vRow = 0;  // first sequence row of the next tile to request
    auto request = [&](uint64_t& next, uint32_t& dst, int& row, const int (&src)[kChunks]) {
        const int valid = L - row < kBN ? L - row : kBN;  // rows of the tile inside the sequence
        if (valid > 0 && row < kEnd) {
            const uint32_t bytes = static_cast<uint32_t>(((valid - 1) * qPitch + kHD) * static_cast<int64_t>(sizeof(T)));
            const u32x4 buf = {static_cast<uint32_t>(next), static_cast<uint32_t>(next >> 32) & 0xffffu, bytes, kRawBufferWord3};
#pragma unroll
            for (int it = 0; it < kChunks; ++it) {
                if (row >= 0 || (waveU * kChunks + it) * 4 >= kBN / 2) loadToLds16(buf, dst + it * 1024, src[it]);
            }
        }
        next += tileStride;
        dst ^= 2 * kTileBytes;
        row += kBN;
    };

    // ---- operand addresses (LDS addresses, the staging area's own included) ----
    // K (A operand of the first product), step st of half h: row 32 h + n, packet 2 st + hh, swizzled by the row.
    // V^T (A operand of the second), block mb, key group u of half h: two transposing reads (see ctxAttnMfma); in each,
    // the lane supplies the address of 4 dims of key row 32 h + 16 u + 8 w + 4 hh + (lane % 16) / 4.
    // The step / block index enters through the swizzle's exclusive-or, on bits the lane's part also uses, so it cannot
    // ride in the instruction's offset field: one register per st and per mb.  They point into the buffers of the tile
    // at hand and change buffers by flipping one bit, once per tile.
    uint32_t kAddr[kHD / 16], vAddr[kHD / 32];
    {
        const int hx = hh ^ (n & 15);
#pragma unroll
        for (int st = 0; st < kHD / 16; ++st) kAddr[st] = ldsBase + n * 256 + (((2 * st) ^ hx) * 16);
        const int g16 = lane / 16, kk = (lane % 16) / 4, qq = lane % 4;
        const int cLo = 2 * (g16 % 2) + qq / 2;
#pragma unroll
        for (int mb = 0; mb < kHD / 32; ++mb) vAddr[mb] = ldsBase + kTileBytes + (4 * hh + kk) * 256 + ((4 * (mb ^ kk) + cLo) * 16) + (qq % 2) * 8;
    }
    // The query fragments must have arrived before the first tile request: a wait for them after it would also wait for
    // the request, which the compiler does not count.
#pragma unroll
    for (int st = 0; st < kHD / 16; ++st) asm volatile("" : "+v"(qf[st]));

    using LdsVec = const __attribute__((address_space(3))) u32x4*;
    using LdsQuad = __attribute__((address_space(3))) s16x4*;
    auto readK = [&](int h, int st) -> u32x4 {  // rows 32 h .. 32 h + 31 of the K tile kAddr points at
        return *reinterpret_cast<LdsVec>(static_cast<uintptr_t>(kAddr[st] + h * 32 * 256));
    };
    auto readV = [&](int h, int f) -> u32x4 {  // fragment f = 4 u + mb of half h of the V tile vAddr points at
        const uintptr_t base = vAddr[f % 4] + (h * 32 + (f / 4) * 16) * 256;
        const s16x4 t0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<LdsQuad>(base));
        const s16x4 t1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<LdsQuad>(base + 8 * 256));
        u32x4 r;
        r[0] = __builtin_bit_cast(u32x2, t0)[0];
        r[1] = __builtin_bit_cast(u32x2, t0)[1];
        r[2] = __builtin_bit_cast(u32x2, t1)[0];
        r[3] = __builtin_bit_cast(u32x2, t1)[1];
        return r;
    };
    auto flipK = [&]() {
#pragma unroll
        for (int st = 0; st < kHD / 16; ++st) kAddr[st] ^= 2 * kTileBytes;
    };
    auto flipV = [&]() {
#pragma unroll
        for (int mb = 0; mb < kHD / 32; ++mb) vAddr[mb] ^= 2 * kTileBytes;
    };

    // exponential of score r of a half; packing of two of them into word w (= r / 2) of the probability fragments
    auto expOne = [&](const f32x16& s, int r) -> float {
        return __builtin_amdgcn_exp2f(s[r]);
    };
    auto packPair = [&](int w, float e0, float e1) -> uint32_t {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef T tx2 __attribute__((ext_vector_type(2)));
        const uint32_t word = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{e0, e1}), tx2));  // one packed conversion
        FragBits<Frag> u;
        u.f = pf[w / 4];
        u.raw[w % 4] = word;
        pf[w / 4] = u.f;
        return word;
    };
    // this lane's maximum over the 16 keys it holds of a half, as a chain of 8 instructions; step i of it
    auto maxStep = [&](const f32x16& s, int i, float m) -> float {
        if (i == 0) return max3(s[0], s[1], s[2]);
        if (i == 7) return max3(m, s[15], s[15]);
        return max3(m, s[2 * i + 1], s[2 * i + 2]);
    };
    // Moves the reference of the lane's query row up by `up`: scales what has been accumulated, shifts the scores of the
    // half at hand.  Rarely taken.
    auto rescale = [&](f32x16& s, float up) {
        const float alpha = __builtin_amdgcn_exp2f(-up);
        lRun *= alpha;
#pragma unroll
        for (int r = 0; r < 16; ++r) negRef[r] -= up;
#pragma unroll
        for (int mb = 0; mb < kHD / 32; ++mb) {
#pragma unroll
            for (int r = 0; r < 16; ++r) o[mb][r] *= alpha;
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] -= up;
    };

    // S^T of the 32 keys in rows 32 h .. of the K tile kAddr points at, into sN, with the exponentials of half sC dealt out
    // between the products (EXP) or nothing in between.
    auto scores = [&](auto expTag, int h, f32x16& sN, const f32x16& sC, const float (&early)[8]) {
        constexpr bool EXP = decltype(expTag)::value;
        u32x4 kf[kKRing];
        float late[8];  // exponentials of scores 8..15, one per step
#pragma unroll
        for (int t = 0; t < kKRing - 1; ++t) kf[t] = readK(h, t);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            if (t + kKRing - 1 < 8) kf[(t + kKRing - 1) % kKRing] = readK(h, t + kKRing - 1);
            if (t == 0) {
                Ops::start(sN, kf[0], qf[0], negRef);
            } else {
                Ops::acc(sN, kf[t % kKRing], qf[t]);
            }
            if constexpr (EXP) {
                // one exponential and one packed conversion per product; scores 0..7 were exponentiated during the
                // products of the phase before (`early`), and a pair is packed two or more steps after its exponentials
                late[t] = expOne(sC, 8 + t);
                if (t < 4) {
                    packPair(t, early[2 * t], early[2 * t + 1]);
                } else if (t < 7) {
                    packPair(t, late[2 * (t - 4)], late[2 * (t - 4) + 1]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (EXP) {
            packPair(7, late[6], late[7]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // O^T += V^T(half h of the tile vAddr points at) . P^T; dealt out between the products (MAX): the row sums of the
    // probabilities at hand and the lane maximum of half sN (returned in tm)
    auto values = [&](auto maxTag, int h, const f32x16& sN, float& tm, float (&early)[8]) {
        constexpr bool MAX = decltype(maxTag)::value;
        u32x4 vf[kVRing];
#pragma unroll
        for (int f = 0; f < kVRing - 1; ++f) vf[f] = readV(h, f);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int f = 0; f < 8; ++f) {
            if (f + kVRing - 1 < 8) vf[(f + kVRing - 1) % kVRing] = readV(h, f + kVRing - 1);
            Ops::acc(o[f % 4], vf[f % kVRing], pf[f / 4]);
            if constexpr (MAX) {
                FragBits<Frag> u;
                u.f = pf[f / 4];
                lRun = Sum::addPair(u.raw[f % 4], lRun);
                // (a product behind: the scores come from matrix instructions the compiler does not see, and a vector
                // instruction may read them only a dozen wait states later)
                if (f >= 1) tm = maxStep(sN, f - 1, tm);
                // the first eight exponentials of the half whose maximum is being taken: should the maximum turn out too
                // high they are thrown away with the rest of the pipeline's state
                if (f >= 1) early[f - 1] = expOne(sN, f - 1);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (MAX) {
            tm = maxStep(sN, 7, tm);
            early[7] = expOne(sN, 7);
        }
    };
    // exponentials of half s into pf, row sums: the unpipelined form
    auto probabilities = [&](const f32x16& s) {
#pragma unroll
        for (int w = 0; w < 8; ++w) lRun = Sum::addPair(packPair(w, expOne(s, 2 * w), expOne(s, 2 * w + 1)), lRun);
    };
    using Yes = std::true_type;
    using No = std::false_type;

    // K tile jt + 1 and V tile jt have landed, every wave has left K tile jt and V tile jt - 1: their buffers take the next ones
    auto top = [&]() {
        waitLdsLoads();
        __syncthreads();
        request(kNext, kDst, kRow, kSrc);
        request(vNext, vDst, vRow, vSrc);
    };

    // ---- prologue: K tile 0; then K tile 1 and V tile 0 travel while the scores of the first 32 keys are computed ----
    request(kNext, kDst, kRow, kSrc);
    waitLdsLoads();
    __syncthreads();
    request(kNext, kDst, kRow, kSrc);
    request(vNext, vDst, vRow, vSrc);
    float tm = 0.f;
    float early[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};  // exponentials of scores 0..7 of the half that is next in line
    if (active) {
        scores(No(), 1, s0, s0, early);
        mfmaSettle(s0);
        if (dg > 0) {  // the first half sets the reference
            float m = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) m = maxStep(s0, i, m);
            rescale(s0, maxWithOtherHalf(m));
#pragma unroll
            for (int r = 0; r < 8; ++r) early[r] = expOne(s0, r);
        }
    }
    flipK();  // from here on kAddr points at K tile jt + 1
    int jt = 0;
    if (active) {
        // A phase that finds the reference too low for some row leaves the pipeline for good: the rest of the wave's
        // tiles go through the plain loop below, which moves the reference where it has to.  With the threshold at
        // 2^kPipeLazyLog2 above the maximum of the wave's first 32 keys that is rare, and the pipelined loop keeps no
        // path on which accumulators are rewritten.  One exit, at the bottom, and the second half of a trip under a
        // condition: with several exits the compiler's loop-exit unification hands every live value through blocks of
        // register copies.
        auto tooLow = [&]() -> bool { return __any(tm > kPipeLazyLog2); };
        int event = 0;
        if (jt < dg) {
            // The wave's priority steps down with the phases.  Of two waves on a SIMD the instruction arbiter serves the older
            // one first (in a loop of nothing but products it gets 85 % of the matrix pipe), so the four older waves of a
            // group reach the next barrier 380 clocks before the four younger ones, which then run alone and less well.  With
            // the steps, a wave that is a phase ahead ranks below its neighbour: 230 clocks, +0.5-1 % on the whole kernel.
            do {
                top();
                __builtin_amdgcn_s_setprio(3);
                scores(Yes(), 0, s1, s0, early);  // phase 1
                __builtin_amdgcn_s_setprio(2);
                values(Yes(), 0, s1, tm, early);  // phase 2
                __builtin_amdgcn_s_setprio(1);
                if (tooLow()) {
                    event = 1;
                } else {
                    scores(Yes(), 1, s0, s1, early);  // phase 3
                    __builtin_amdgcn_s_setprio(0);
                    values(Yes(), 1, s0, tm, early);  // phase 4
                    flipK();
                    flipV();
                    ++jt;
                    // the unmasked maximum of the diagonal tile must not move the reference: its turn comes below
                    if (jt < dg && tooLow()) event = 2;
                }
            } while (jt < dg && event == 0);
            __builtin_amdgcn_s_setprio(0);
        }
        // the row's maximum over the 32 keys of half s; moves the reference when it is more than the lazy margin above it
        auto settleHalf = [&](f32x16& s) {
            mfmaSettle(s);
            float m = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) m = maxStep(s, i, m);
            if (__any(m > kLazyLog2)) rescale(s, fmaxf(maxWithOtherHalf(m), 0.f));
        };
        float unused = 0.f;
        float unusedEarly[8];
        if (event == 1) {  // the upper half of tile jt is still to do
            settleHalf(s1);
            probabilities(s1);
            values(No(), 1, s1, unused, unusedEarly);
            scores(No(), 1, s0, s0, unusedEarly);
            flipK();
            flipV();
            ++jt;
        }
        if (event != 0) {
            while (jt < dg) {  // s0 holds the lower half of tile jt, not yet looked at
                top();
                settleHalf(s0);
                probabilities(s0);
                values(No(), 0, s0, unused, unusedEarly);
                scores(No(), 0, s1, s1, unusedEarly);
                settleHalf(s1);
                probabilities(s1);
                values(No(), 1, s1, unused, unusedEarly);
                scores(No(), 1, s0, s0, unusedEarly);
                flipK();
                flipV();
                ++jt;
            }
        }
        // ---- the diagonal tile: mask, maximum, exponentials, second product, nothing overlapped.  A wave whose rows are
        // the lower 32 of its tile's 64 sees only the lower half of the keys. ----
        top();
        const bool both = (waveRowLo & 32) != 0;
        if (both) scores(No(), 0, s1, s1, unusedEarly);
        mfmaSettle(s0, s1);  // the masks below overwrite what the last products wrote
        mfmaSettle(o[0], o[1], o[2], o[3]);
        const int key0 = dg * kBN;
        const int row = waveRowLo + n;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int key = key0 + 8 * (r / 4) + 4 * hh + r % 4;
            if (key > row) s0[r] = -1e30f;
            if (!both || key + 32 > row) s1[r] = -1e30f;
        }
        float m = 0.f, m1 = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            m = maxStep(s0, i, m);
            m1 = maxStep(s1, i, m1);
        }
        float up = maxWithOtherHalf(fmaxf(m, m1));
        const bool first = dg == 0;
        if (first || __any(up > kLazyLog2)) {
            if (!first) up = fmaxf(up, 0.f);
#pragma unroll
            for (int r = 0; r < 16; ++r) s1[r] -= up;
            rescale(s0, up);
        }
        probabilities(s0);
        values(No(), 0, s0, unused, unusedEarly);
        if (both) {
            probabilities(s1);
            values(No(), 1, s1, unused, unusedEarly);
        }
        ++jt;
    }
    mfmaSettle(o[0], o[1], o[2], o[3]);
    for (; jt < numKeyTiles; ++jt) top();  // the other waves' remaining tiles: this wave only fetches its share

    // ---- normalise, transpose through LDS, write rows with 16-byte stores ----
    const float lTot = lRun + __shfl_xor(lRun, 32, kWave);
    const float inv = 1.0f / lTot;
    waitLdsLoads();
    __syncthreads();  // the K/V tiles are dead and no request is in flight; reuse the storage as a [BM][kLD] output tile
    T* sO = smem;
#pragma unroll
    for (int mb = 0; mb < kHD / 32; ++mb) {
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
            // registers 4 rq .. 4 rq + 3 of o[mb] are dims 32 mb + 8 rq + 4 hh .. + 3
            T pk[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) pk[e] = static_cast<T>(o[mb][4 * rq + e] * inv);
            *reinterpret_cast<u32x2*>(sO + (wave * 32 + n) * kLD + 32 * mb + 8 * rq + 4 * hh) = *reinterpret_cast<const u32x2*>(pk);
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    T* oBase = out + seqStart * qPitch + static_cast<int64_t>(head) * kHD;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const int id = it * kWave + lane;
        const int row = id / 16;
        const int c = id % 16;
        const int grow = m0 + wave * 32 + row;
        if (grow < L) {
            const u32x4 val = *reinterpret_cast<const u32x4*>(sO + (wave * 32 + row) * kLD + c * 8);
            *reinterpret_cast<u32x4*>(oBase + grow * qPitch + c * 8) = val;
        }
    }
}

// Any dtype / head size up to 512: one wave per (query row, head); lanes split the head dimension.
template <typename T, typename AccT>
__global__ __launch_bounds__(kWave) void ctxAttnGeneric(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, CtxArgs a,
                                                        int D, AccT scale) {
    constexpr int kPerLane = 8;
    const int head = blockIdx.y;
    const int64_t grow = blockIdx.x;  // row of the packed tensors
    // find the sequence that owns this row
    int seq = 0;
    SeqInfo si{0, 0};
    for (; seq < a.batch; ++seq) {
        si = loadSeq(a, seq);
        if (grow >= si.start && grow < si.start + si.len) break;
    }
    if (seq >= a.batch) return;
    const int64_t r = grow - si.start;
    const int lane = threadIdx.x;
    const int64_t qPitch = static_cast<int64_t>(a.H) * D;
    const int64_t rowPitch = static_cast<int64_t>(a.H / a.G) * D;  // k and v
    const int kvHead = head / a.G;
    const T* qRow = q + grow * qPitch + static_cast<int64_t>(head) * D;
    AccT qv[kPerLane], acc[kPerLane];
#pragma unroll
    for (int e = 0; e < kPerLane; ++e) {
        const int d = lane + e * kWave;
        qv[e] = d < D ? static_cast<AccT>(qRow[d]) : static_cast<AccT>(0);
        acc[e] = 0;
    }
    AccT m = static_cast<AccT>(-INFINITY), l = 0;
    const int64_t jLast = a.causal ? r : si.len - 1;
    for (int64_t j = 0; j <= jLast; ++j) {
        const T* kRow = k + (si.start + j) * rowPitch + static_cast<int64_t>(kvHead) * D;
        const T* vRow = v + (si.start + j) * rowPitch + static_cast<int64_t>(kvHead) * D;
        AccT part = 0;
#pragma unroll
        for (int e = 0; e < kPerLane; ++e) {
            const int d = lane + e * kWave;
            if (d < D) part += qv[e] * static_cast<AccT>(kRow[d]);
        }
        const AccT sc = waveSum(part) * scale;
        const AccT mNew = sc > m ? sc : m;
        const AccT alpha = static_cast<AccT>(exp(static_cast<double>(m - mNew)));
        const AccT p = static_cast<AccT>(exp(static_cast<double>(sc - mNew)));
        l = l * alpha + p;
#pragma unroll
        for (int e = 0; e < kPerLane; ++e) {
            const int d = lane + e * kWave;
            if (d < D) acc[e] = acc[e] * alpha + p * static_cast<AccT>(vRow[d]);
        }
        m = mNew;
    }
    T* oRow = out + grow * qPitch + static_cast<int64_t>(head) * D;
#pragma unroll
    for (int e = 0; e < kPerLane; ++e) {
        const int d = lane + e * kWave;
        if (d < D) oRow[d] = static_cast<T>(acc[e] / l);
    }
    if (a.lse != nullptr && lane == 0 && r < a.lseStride)
        a.lse[(static_cast<int64_t>(seq) * a.H + head) * a.lseStride + r] = static_cast<float>(static_cast<double>(m) + log(static_cast<double>(l)));
}

template <typename T, int NWV, bool GEN = false>
diopiError_t launchMfma(diopiContextHandle_t ctx, hipStream_t stream, void* out, const void* q, const void* k, const void* v, CtxArgs a,
                        const PlanStore& store) {
    constexpr int BM = NWV * 32;
    a.tilesBound = static_cast<int>(ceilDiv(a.rows, BM)) + a.batch;
    const int64_t total = static_cast<int64_t>(a.tilesBound) * a.H;
    ROCM_CHECK(total < INT32_MAX / 2, "context attention: too many tiles for one launch");
    a.totalItems = static_cast<int>(total);
    // visiting order of the query tiles, rebuilt by every call on the device: context-owned scratch, or the library's
    // static array when the caller must not allocate
    void* planMem = store.fixed;
    if (store.fixed != nullptr) {
        ROCM_CHECK(a.tilesBound <= store.capacity,
                   "the allocation-free entry point holds a plan of at most %d query tiles of %d rows (+ one per sequence); this call needs %d",
                   store.capacity, BM, a.tilesBound);
    } else {
        ROCM_CALL(requireScratch(ctx, static_cast<int64_t>(a.tilesBound) * sizeof(int4), &planMem));
    }
    a.plan = static_cast<const int4*>(planMem);
    const int maxTiles = static_cast<int>(ceilDiv(a.rows, BM));
    const size_t planLds = (4 * static_cast<size_t>(a.batch) + maxTiles) * sizeof(int);
    hipLaunchKernelGGL(ctxAttnPlan, dim3(1), dim3(kPlanThreads), planLds, stream, static_cast<int4*>(planMem), a, maxTiles, BM);
    ROCM_LAUNCH_CHECK();
    const int grid = static_cast<int>(ceilDiv(total, kNumXcd)) * kNumXcd;
    constexpr int kStaging = 2 * 2 * kBN * kHD, kOutTile = BM * kLD;  // elements: two (K, V) buffers; the output tile that reuses them
    constexpr int ldsBytes = (kStaging > kOutTile ? kStaging : kOutTile) * static_cast<int>(sizeof(T));
    ROCM_CALL(grantDynamicLds(reinterpret_cast<const void*>(ctxAttnMfma<T, NWV, GEN>), ldsBytes));
    if constexpr (!GEN) {  // the lightllm operator: causal, one key/value head per query head, the literal scale
        ROCM_CALL(grantDynamicLds(reinterpret_cast<const void*>(ctxAttnPipe<T, NWV>), ldsBytes));
        hipLaunchKernelGGL((ctxAttnPipe<T, NWV>), dim3(grid), dim3(NWV * kWave), ldsBytes, stream, static_cast<T*>(out), static_cast<const T*>(q),
                           static_cast<const T*>(k), static_cast<const T*>(v), a);
        ROCM_LAUNCH_CHECK();
        return diopiSuccess;
    }
    hipLaunchKernelGGL((ctxAttnMfma<T, NWV, GEN>), dim3(grid), dim3(NWV * kWave), ldsBytes, stream, static_cast<T*>(out), static_cast<const T*>(q),
                       static_cast<const T*>(k), static_cast<const T*>(v), a);
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
}

template <typename T, typename AccT>
diopiError_t launchGeneric(hipStream_t stream, void* out, const void* q, const void* k, const void* v, const CtxArgs& a, int D, double softmaxScale) {
    ROCM_CHECK(D <= 8 * kWave, "context attention: head size %d is not supported (at most %d)", D, 8 * kWave);
    ROCM_CHECK(a.H <= 65535, "context attention: %d heads exceed the launch limit", a.H);
    ROCM_CHECK(a.rows <= INT32_MAX, "context attention: too many rows for one launch");
    const AccT scale = static_cast<AccT>(softmaxScale);
    hipLaunchKernelGGL((ctxAttnGeneric<T, AccT>), dim3(static_cast<unsigned>(a.rows), static_cast<unsigned>(a.H)), dim3(kWave), 0, stream,
                       static_cast<T*>(out), static_cast<const T*>(q), static_cast<const T*>(k), static_cast<const T*>(v), a, D, scale);
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
}

// Picks the kernel for one call: the matrix-core kernel for 16-bit tensors with head size 128 (4 waves per query tile
// of 128 rows, or 8 waves per 256 rows once the sequences are long enough to fill them), the one-wave-per-row kernel
// for everything else.  Returns diopiDtypeNotSupported (without a message) for a dtype no kernel takes.
template <bool GEN>
diopiError_t dispatchAttention(diopiContextHandle_t ctx, hipStream_t stream, const TensorView& vOut, const TensorView& vQ, const TensorView& vK,
                               const TensorView& vV, const CtxArgs& a, int D, double softmaxScale, const PlanStore& store = PlanStore()) {
    const bool aligned =
        ((reinterpret_cast<uintptr_t>(vQ.data) | reinterpret_cast<uintptr_t>(vK.data) | reinterpret_cast<uintptr_t>(vV.data) | reinterpret_cast<uintptr_t>(vOut.data)) & 15) == 0;
    // the planning kernel keeps two ints per sequence and one per query tile in LDS
    const bool planFits = (4 * static_cast<int64_t>(a.batch) + a.rows / kBMMin + 1) * 4 <= 64 * 1024 && a.rows <= INT32_MAX;
    // the tile requests address a 64-row tile with 32-bit byte offsets
    const bool tileFits = static_cast<int64_t>(a.H) * kHD * 8 * kBN < INT32_MAX;
    const bool fast = D == kHD && aligned && planFits && tileFits;
    // 256-row query tiles (8 waves share each K/V tile) once the sequences are long enough to fill them
    const bool wide = a.rows >= 1024 * static_cast<int64_t>(a.batch);
    switch (vQ.dtype) {
        case diopi_dtype_float16:
            return fast ? (wide ? launchMfma<half_t, 8, GEN>(ctx, stream, vOut.data, vQ.data, vK.data, vV.data, a, store)
                                : launchMfma<half_t, 4, GEN>(ctx, stream, vOut.data, vQ.data, vK.data, vV.data, a, store))
                        : launchGeneric<half_t, float>(stream, vOut.data, vQ.data, vK.data, vV.data, a, D, softmaxScale);
        case diopi_dtype_bfloat16:
            return fast ? (wide ? launchMfma<bf16_t, 8, GEN>(ctx, stream, vOut.data, vQ.data, vK.data, vV.data, a, store)
                                : launchMfma<bf16_t, 4, GEN>(ctx, stream, vOut.data, vQ.data, vK.data, vV.data, a, store))
                        : launchGeneric<bf16_t, float>(stream, vOut.data, vQ.data, vK.data, vV.data, a, D, softmaxScale);
        case diopi_dtype_float32: return launchGeneric<float, float>(stream, vOut.data, vQ.data, vK.data, vV.data, a, D, softmaxScale);
        case diopi_dtype_float64: return launchGeneric<double, double>(stream, vOut.data, vQ.data, vK.data, vV.data, a, D, softmaxScale);
        default: break;
    }
    return diopiDtypeNotSupported;
}

}  // namespace
}  // namespace rocm

namespace rocm {
namespace {

// Device address of the static plan array on the current device.  In host code the array's name is only a stand-in
// for the symbol; the address a kernel may use comes from hipGetSymbolAddress, once per device (each device holds its
// own copy at its own address).
diopiError_t staticPlanStore(PlanStore* store) {
    constexpr int kMaxDevices = 64;
    static std::mutex mtx;
    static int4* address[kMaxDevices] = {nullptr};
    int dev = 0;
    ROCM_HIP(hipGetDevice(&dev));
    ROCM_CHECK(dev >= 0 && dev < kMaxDevices, "device index %d is beyond the %d devices the allocation-free entry point keeps a plan for", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(mtx);
    if (address[dev] == nullptr) {
        void* ptr = nullptr;
        ROCM_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        ROCM_CHECK(ptr != nullptr, "hipGetSymbolAddress returned no address for the static plan array");
        address[dev] = static_cast<int4*>(ptr);
    }
    store->fixed = address[dev];
    store->capacity = kStaticPlanEntries;
    return diopiSuccess;
}

// diopiContextAttentionInference and its allocation-free variant: the same checks and kernels, the tile plan in the
// context's scratch (`staticPlan` false) or in the library's static array.
diopiError_t contextAttention(diopiContextHandle_t ctx, diopiTensorHandle_t context_attention_out, diopiConstTensorHandle_t q, diopiConstTensorHandle_t k,
                              diopiConstTensorHandle_t v, diopiConstTensorHandle_t b_start_loc, diopiConstTensorHandle_t b_seq_len, bool staticPlan) {
    TensorView vOut, vQ, vK, vV, vStart, vLen;
    ROCM_CALL(unwrap(context_attention_out, "context_attention_out", &vOut));
    ROCM_CALL(unwrap(q, "q", &vQ));
    ROCM_CALL(unwrap(k, "k", &vK));
    ROCM_CALL(unwrap(v, "v", &vV));
    ROCM_CALL(unwrap(b_start_loc, "b_start_loc", &vStart));
    ROCM_CALL(unwrap(b_seq_len, "b_seq_len", &vLen));
    ROCM_CALL(requireDeviceContiguous(vOut, "context_attention_out"));
    ROCM_CALL(requireDeviceContiguous(vQ, "q"));
    ROCM_CALL(requireDeviceContiguous(vK, "k"));
    ROCM_CALL(requireDeviceContiguous(vV, "v"));
    ROCM_CALL(requireDeviceContiguous(vStart, "b_start_loc"));
    ROCM_CALL(requireDeviceContiguous(vLen, "b_seq_len"));
    ROCM_CHECK(vQ.ndim == 3, "q must be [rows, heads, head_dim], got rank %d", vQ.ndim);
    ROCM_CHECK(vK.sameShape(vQ) && vV.sameShape(vQ) && vOut.sameShape(vQ), "q, k, v and out must have identical shapes (the reference has no grouped heads here)");
    ROCM_CHECK(isFloatDtype(vQ.dtype) && vK.dtype == vQ.dtype && vV.dtype == vQ.dtype && vOut.dtype == vQ.dtype,
               "q, k, v and out must share one floating dtype (q is %s)", dtypeName(vQ.dtype));
    ROCM_CHECK(vStart.ndim == 1 && vLen.ndim == 1 && vStart.shape[0] == vLen.shape[0], "b_start_loc and b_seq_len must be 1-D of equal length");
    ROCM_CHECK(isIndexDtype(vStart.dtype) && isIndexDtype(vLen.dtype), "b_start_loc and b_seq_len must be int32 or int64");
    ROCM_CHECK(vStart.shape[0] <= 65535 && vQ.shape[1] <= INT32_MAX / 1024 && vQ.shape[2] <= 65535, "batch / head count / head size out of range");
    if (vQ.numel == 0 || vStart.shape[0] == 0) return diopiSuccess;

    CtxArgs a;
    a.bStartLoc = vStart.data;
    a.bSeqLen = vLen.data;
    a.start64 = vStart.dtype == diopi_dtype_int64;
    a.len64 = vLen.dtype == diopi_dtype_int64;
    a.batch = static_cast<int>(vStart.shape[0]);
    a.H = static_cast<int>(vQ.shape[1]);
    a.rows = vQ.shape[0];
    a.tilesBound = 0;
    a.totalItems = 0;
    a.cumulative = false;
    a.uniformLen = 0;
    a.causal = true;
    a.G = 1;
    a.scaleLog2 = 0.f;
    a.lse = nullptr;
    a.lseStride = 0;
    const int D = static_cast<int>(vQ.shape[2]);
    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    PlanStore store;
    if (staticPlan) ROCM_CALL(staticPlanStore(&store));
    const diopiError_t err = dispatchAttention<false>(ctx, stream, vOut, vQ, vK, vV, a, D, 1.0 / std::sqrt(static_cast<double>(D)), store);
    if (err != diopiDtypeNotSupported) return err;
    setLastError("diopiContextAttentionInference: dtype %s is not supported", dtypeName(vQ.dtype));
    return diopiDtypeNotSupported;
}

}  // namespace
}  // namespace rocm

extern "C" diopiError_t diopiContextAttentionInference(diopiContextHandle_t ctx, diopiTensorHandle_t context_attention_out, diopiConstTensorHandle_t q,
                                                       diopiConstTensorHandle_t k, diopiConstTensorHandle_t v, diopiConstTensorHandle_t b_start_loc,
                                                       diopiConstTensorHandle_t b_seq_len, int max_input_len) {
    ROCM_ENTRY_BEGIN
    (void)max_input_len;  // never read by the reference (functions_lightllm.cpp:127-147); lengths come from b_seq_len
    return rocm::contextAttention(ctx, context_attention_out, q, k, v, b_start_loc, b_seq_len, false);
    ROCM_ENTRY_END
}

// The same operator for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that
// forbid hipMalloc): it calls neither diopiRequireBuffer / diopiRequireTensor nor any allocating routine.  The tile
// plan lives in a static device array of kStaticPlanEntries entries that all such calls on one device share: calls
// that overlap on one device (two streams) race on it.  Nothing in it has to start at zero: the planning kernel
// rewrites every entry a call reads.  Inputs beyond the array's capacity are rejected with an error.
extern "C" diopiError_t diopiContextAttentionInferenceNoAlloc(diopiContextHandle_t ctx, diopiTensorHandle_t context_attention_out,
                                                              diopiConstTensorHandle_t q, diopiConstTensorHandle_t k, diopiConstTensorHandle_t v,
                                                              diopiConstTensorHandle_t b_start_loc, diopiConstTensorHandle_t b_seq_len, int max_input_len) {
    ROCM_ENTRY_BEGIN
    (void)max_input_len;
    return rocm::contextAttention(ctx, context_attention_out, q, k, v, b_start_loc, b_seq_len, true);
    ROCM_ENTRY_END
}

namespace rocm {
namespace {

// Variable-length attention behind diopiFlashAttentionVarLen and diopiMultiHeadAttentionVarLen.
diopiError_t attentionVarLen(diopiContextHandle_t ctx, const char* opName, diopiTensorHandle_t attention_out, diopiTensorHandle_t softmax_lse,
                             diopiConstTensorHandle_t q, diopiConstTensorHandle_t k, diopiConstTensorHandle_t v, diopiConstTensorHandle_t cum_seq_q,
                             diopiConstTensorHandle_t cum_seq_kv, int64_t max_seqlen_q, double softmax_scale, bool is_causal) {
    TensorView vOut, vQ, vK, vV, vCuQ, vCuK, vLse;
    ROCM_CALL(unwrap(attention_out, "attention_out", &vOut));
    ROCM_CALL(unwrap(q, "q", &vQ));
    ROCM_CALL(unwrap(k, "k", &vK));
    ROCM_CALL(unwrap(v, "v", &vV));
    ROCM_CALL(unwrap(cum_seq_q, "cum_seq_q", &vCuQ));
    ROCM_CALL(unwrap(cum_seq_kv, "cum_seq_kv", &vCuK));
    ROCM_CALL(requireDeviceContiguous(vOut, "attention_out"));
    ROCM_CALL(requireDeviceContiguous(vQ, "q"));
    ROCM_CALL(requireDeviceContiguous(vK, "k"));
    ROCM_CALL(requireDeviceContiguous(vV, "v"));
    ROCM_CALL(requireDeviceContiguous(vCuQ, "cum_seq_q"));
    ROCM_CALL(requireDeviceContiguous(vCuK, "cum_seq_kv"));
    const bool haveLse = softmax_lse != nullptr;
    if (haveLse) {
        ROCM_CALL(unwrap(softmax_lse, "softmax_lse", &vLse));
        ROCM_CALL(requireDeviceContiguous(vLse, "softmax_lse"));
    }
    ROCM_CHECK(vQ.ndim == 3 && vK.ndim == 3, "q and k must be [tokens, heads, head_dim], got ranks %d and %d", vQ.ndim, vK.ndim);
    ROCM_CHECK(vOut.sameShape(vQ) && vV.sameShape(vK), "attention_out must have the shape of q, v the shape of k");
    // like the reference's statement (customized_test.py:550), queries and keys of a sequence are the same tokens
    ROCM_CHECK(vK.shape[0] == vQ.shape[0] && vK.shape[2] == vQ.shape[2], "q and k must have the same token count and head size");
    ROCM_CHECK(vK.shape[1] > 0 && vQ.shape[1] % vK.shape[1] == 0, "the %lld query heads must be a multiple of the %lld key/value heads",
               static_cast<long long>(vQ.shape[1]), static_cast<long long>(vK.shape[1]));
    ROCM_CHECK(isFloatDtype(vQ.dtype) && vK.dtype == vQ.dtype && vV.dtype == vQ.dtype && vOut.dtype == vQ.dtype,
               "q, k, v and attention_out must share one floating dtype (q is %s)", dtypeName(vQ.dtype));
    ROCM_CHECK(vCuQ.ndim == 1 && vCuQ.shape[0] >= 1 && vCuK.ndim == 1 && vCuK.shape[0] == vCuQ.shape[0] && isIndexDtype(vCuQ.dtype) &&
                   vCuK.dtype == vCuQ.dtype,
               "cum_seq_q and cum_seq_kv must be 1-D int32 or int64 tensors of batch + 1 entries");
    ROCM_CHECK(vCuQ.shape[0] - 1 <= 65535 && vQ.shape[1] <= INT32_MAX / 1024 && vQ.shape[2] <= 65535, "batch / head count / head size out of range");
    ROCM_CHECK(max_seqlen_q >= 0 && max_seqlen_q <= INT32_MAX, "max_seqlen_q out of range");
    const int64_t batch = vCuQ.shape[0] - 1;
    if (haveLse) {
        ROCM_CHECK(vLse.dtype == diopi_dtype_float32 && vLse.numel == batch * vQ.shape[1] * static_cast<int64_t>(max_seqlen_q),
                   "softmax_lse must be float32 [batch, heads, max_seqlen_q] = [%lld, %lld, %lld]", static_cast<long long>(batch),
                   static_cast<long long>(vQ.shape[1]), static_cast<long long>(max_seqlen_q));
    }
    if (vQ.numel == 0 || batch == 0) return diopiSuccess;

    CtxArgs a;
    a.bStartLoc = vCuQ.data;
    a.bSeqLen = nullptr;
    a.start64 = vCuQ.dtype == diopi_dtype_int64;
    a.len64 = a.start64;
    a.batch = static_cast<int>(batch);
    a.H = static_cast<int>(vQ.shape[1]);
    a.rows = vQ.shape[0];
    a.tilesBound = 0;
    a.totalItems = 0;
    a.cumulative = true;
    a.uniformLen = 0;
    a.causal = is_causal;
    a.G = static_cast<int>(vQ.shape[1] / vK.shape[1]);
    const int D = static_cast<int>(vQ.shape[2]);
    // the Python layer passes 1/sqrt(head_dim) for "None" (diopi_functions.py:7564-7566); zero means the same here
    const double scale = softmax_scale != 0.0 ? softmax_scale : 1.0 / std::sqrt(static_cast<double>(D));
    a.scaleLog2 = static_cast<float>(scale * 1.4426950408889634);
    a.lse = haveLse ? static_cast<float*>(vLse.data) : nullptr;
    a.lseStride = static_cast<int>(max_seqlen_q);
    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    const diopiError_t err = dispatchAttention<true>(ctx, stream, vOut, vQ, vK, vV, a, D, scale);
    if (err != diopiDtypeNotSupported) return err;
    setLastError("%s: dtype %s is not supported", opName, dtypeName(vQ.dtype));
    return diopiDtypeNotSupported;
}

// Attention on padded batches behind diopiFlashAttention and diopiMultiHeadAttention.
diopiError_t attentionPadded(diopiContextHandle_t ctx, const char* opName, diopiTensorHandle_t attention_out, diopiTensorHandle_t softmax_lse,
                             diopiConstTensorHandle_t q, diopiConstTensorHandle_t k, diopiConstTensorHandle_t v, double softmax_scale, bool is_causal) {
    TensorView vOut, vQ, vK, vV, vLse;
    ROCM_CALL(unwrap(attention_out, "attention_out", &vOut));
    ROCM_CALL(unwrap(q, "q", &vQ));
    ROCM_CALL(unwrap(k, "k", &vK));
    ROCM_CALL(unwrap(v, "v", &vV));
    ROCM_CALL(requireDeviceContiguous(vOut, "attention_out"));
    ROCM_CALL(requireDeviceContiguous(vQ, "q"));
    ROCM_CALL(requireDeviceContiguous(vK, "k"));
    ROCM_CALL(requireDeviceContiguous(vV, "v"));
    const bool haveLse = softmax_lse != nullptr;
    if (haveLse) {
        ROCM_CALL(unwrap(softmax_lse, "softmax_lse", &vLse));
        ROCM_CALL(requireDeviceContiguous(vLse, "softmax_lse"));
    }
    ROCM_CHECK(vQ.ndim == 4 && vK.ndim == 4, "q and k must be [batch, seq_len, heads, head_dim], got ranks %d and %d", vQ.ndim, vK.ndim);
    ROCM_CHECK(vOut.sameShape(vQ) && vV.sameShape(vK), "attention_out must have the shape of q, v the shape of k");
    // like the reference's statement (customized_test.py:473-481: one seqlen for the mask), queries and keys are the same positions
    ROCM_CHECK(vK.shape[0] == vQ.shape[0] && vK.shape[1] == vQ.shape[1] && vK.shape[3] == vQ.shape[3],
               "q and k must have the same batch size, sequence length and head size");
    ROCM_CHECK(vK.shape[2] > 0 && vQ.shape[2] % vK.shape[2] == 0, "the %lld query heads must be a multiple of the %lld key/value heads",
               static_cast<long long>(vQ.shape[2]), static_cast<long long>(vK.shape[2]));
    ROCM_CHECK(isFloatDtype(vQ.dtype) && vK.dtype == vQ.dtype && vV.dtype == vQ.dtype && vOut.dtype == vQ.dtype,
               "q, k, v and attention_out must share one floating dtype (q is %s)", dtypeName(vQ.dtype));
    ROCM_CHECK(vQ.shape[0] <= 65535 && vQ.shape[1] <= INT32_MAX && vQ.shape[2] <= INT32_MAX / 1024 && vQ.shape[3] <= 65535,
               "batch / sequence length / head count / head size out of range");
    if (haveLse) {
        ROCM_CHECK(vLse.dtype == diopi_dtype_float32 && vLse.numel == vQ.shape[0] * vQ.shape[2] * vQ.shape[1],
                   "softmax_lse must be float32 [batch, heads, seq_len] = [%lld, %lld, %lld]", static_cast<long long>(vQ.shape[0]),
                   static_cast<long long>(vQ.shape[2]), static_cast<long long>(vQ.shape[1]));
    }
    if (vQ.numel == 0) return diopiSuccess;

    CtxArgs a;
    a.bStartLoc = nullptr;
    a.bSeqLen = nullptr;
    a.start64 = false;
    a.len64 = false;
    a.batch = static_cast<int>(vQ.shape[0]);
    a.H = static_cast<int>(vQ.shape[2]);
    a.rows = vQ.shape[0] * vQ.shape[1];
    a.tilesBound = 0;
    a.totalItems = 0;
    a.cumulative = false;
    a.uniformLen = static_cast<int>(vQ.shape[1]);
    a.causal = is_causal;
    a.G = static_cast<int>(vQ.shape[2] / vK.shape[2]);
    const int D = static_cast<int>(vQ.shape[3]);
    const double scale = softmax_scale != 0.0 ? softmax_scale : 1.0 / std::sqrt(static_cast<double>(D));
    a.scaleLog2 = static_cast<float>(scale * 1.4426950408889634);
    a.lse = haveLse ? static_cast<float*>(vLse.data) : nullptr;
    a.lseStride = static_cast<int>(vQ.shape[1]);
    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    // the kernels see the packed [batch * seq_len, heads, head_dim] view
    TensorView pq = vQ, pk = vK, pv = vV, po = vOut;
    const diopiError_t err = dispatchAttention<true>(ctx, stream, po, pq, pk, pv, a, D, scale);
    if (err != diopiDtypeNotSupported) return err;
    setLastError("%s: dtype %s is not supported", opName, dtypeName(vQ.dtype));
    return diopiDtypeNotSupported;
}

}  // namespace
}  // namespace rocm

extern "C" diopiError_t diopiFlashAttentionVarLen(diopiContextHandle_t ctx, diopiTensorHandle_t attention_out, diopiTensorHandle_t softmax_lse,
                                                  diopiGeneratorHandle_t gen, diopiConstTensorHandle_t q, diopiConstTensorHandle_t k, diopiConstTensorHandle_t v,
                                                  diopiConstTensorHandle_t cum_seq_q, diopiConstTensorHandle_t cum_seq_kv, diopiConstTensorHandle_t alibi_slopes,
                                                  int32_t max_seqlen_q, int32_t max_seqlen_kv, float p_dropout, float softmax_scale, bool is_causal,
                                                  int32_t window_size_left, int32_t window_size_right) {
    ROCM_ENTRY_BEGIN
    using namespace rocm;
    (void)gen;            // only dropout draws random numbers
    (void)max_seqlen_kv;  // lengths come from the cumulative tensors
    // the reference's statement covers neither of these (customized_test.py:540 "TODO: impl for alibi and sliding window")
    if (p_dropout != 0.f || alibi_slopes != nullptr || window_size_left >= 0 || window_size_right >= 0) {
        setLastError("diopiFlashAttentionVarLen: dropout, ALiBi slopes and sliding windows are not implemented");
        return diopiNoImplement;
    }
    return attentionVarLen(ctx, "diopiFlashAttentionVarLen", attention_out, softmax_lse, q, k, v, cum_seq_q, cum_seq_kv, max_seqlen_q, softmax_scale,
                           is_causal);
    ROCM_ENTRY_END
}

extern "C" diopiError_t diopiFlashAttention(diopiContextHandle_t ctx, diopiTensorHandle_t attention_out, diopiTensorHandle_t softmax_lse,
                                            diopiGeneratorHandle_t gen, diopiConstTensorHandle_t q, diopiConstTensorHandle_t k, diopiConstTensorHandle_t v,
                                            diopiConstTensorHandle_t alibi_slopes, float p_dropout, float softmax_scale, bool is_causal,
                                            int32_t window_size_left, int32_t window_size_right) {
    ROCM_ENTRY_BEGIN
    using namespace rocm;
    (void)gen;  // only dropout draws random numbers
    // the reference's statement covers neither of these (customized_test.py:463 "TODO: impl for alibi and sliding window")
    if (p_dropout != 0.f || alibi_slopes != nullptr || window_size_left >= 0 || window_size_right >= 0) {
        setLastError("diopiFlashAttention: dropout, ALiBi slopes and sliding windows are not implemented");
        return diopiNoImplement;
    }
    return attentionPadded(ctx, "diopiFlashAttention", attention_out, softmax_lse, q, k, v, softmax_scale, is_causal);
    ROCM_ENTRY_END
}

// The two older names of the same operators (proto/include/diopi/functions_ext.h:93-95 and 150-153, "deprecated: use
// diopiFlashAttention / diopiFlashAttentionVarLen instead"; Python statements customized_test.py:416-460).  No grouped
// heads in their statement, but nothing here depends on that.  The debug mask only exists with dropout.
extern "C" diopiError_t diopiMultiHeadAttention(diopiContextHandle_t ctx, diopiTensorHandle_t q, diopiTensorHandle_t k, diopiTensorHandle_t v, double dropout_p,
                                                bool is_causal, bool return_debug_mask, double scale, diopiTensorHandle_t out, diopiTensorHandle_t softmax_lse,
                                                diopiGeneratorHandle_t gen, diopiTensorHandle_t debug_attn_mask) {
    ROCM_ENTRY_BEGIN
    using namespace rocm;
    (void)gen;
    (void)debug_attn_mask;
    if (dropout_p != 0.0 || return_debug_mask) {
        setLastError("diopiMultiHeadAttention: dropout and its debug mask are not implemented");
        return diopiNoImplement;
    }
    return attentionPadded(ctx, "diopiMultiHeadAttention", out, softmax_lse, q, k, v, scale, is_causal);
    ROCM_ENTRY_END
}

extern "C" diopiError_t diopiMultiHeadAttentionVarLen(diopiContextHandle_t ctx, diopiTensorHandle_t q, diopiTensorHandle_t k, diopiTensorHandle_t v,
                                                      diopiConstTensorHandle_t cum_seq_q, diopiConstTensorHandle_t cum_seq_k, int64_t max_q, int64_t max_k,
                                                      double dropout_p, bool is_causal, bool return_debug_mask, double scale, diopiTensorHandle_t out,
                                                      diopiTensorHandle_t softmax_lse, diopiGeneratorHandle_t gen, diopiTensorHandle_t debug_attn_mask) {
    ROCM_ENTRY_BEGIN
    using namespace rocm;
    (void)gen;
    (void)debug_attn_mask;
    (void)max_k;
    if (dropout_p != 0.0 || return_debug_mask) {
        setLastError("diopiMultiHeadAttentionVarLen: dropout and its debug mask are not implemented");
        return diopiNoImplement;
    }
    return attentionVarLen(ctx, "diopiMultiHeadAttentionVarLen", out, softmax_lse, q, k, v, cum_seq_q, cum_seq_k, max_q, scale, is_causal);
    ROCM_ENTRY_END
}

// Causal prefill on a padded batch with flattened heads (proto/include/diopi/functions_ext.h:684-686; Python statement
// customized_test.py:751-780): query and out are [batch * max_input_len, num_heads * dim], key and value
// [batch * max_input_len, num_kv_heads * dim]; sequence i owns rows [i * max_input_len, (i + 1) * max_input_len) and
// every row attends to the rows of its sequence up to its own.  Like the statement, this takes only the batch size
// from actual_seq_lengths and computes every row (under the causal mask the rows inside a shorter actual length do
// not depend on the padding behind them), and it does not read atten_mask: the statement builds the lower-triangular
// mask itself.
extern "C" diopiError_t diopiPromptFlashAttention(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t query,
                                                  diopiConstTensorHandle_t key, diopiConstTensorHandle_t value, diopiConstTensorHandle_t atten_mask,
                                                  diopiSize_t actual_seq_lengths, int64_t max_input_len, int64_t num_heads, int64_t num_kv_heads, int64_t dim) {
    ROCM_ENTRY_BEGIN
    using namespace rocm;
    (void)atten_mask;
    TensorView vOut, vQ, vK, vV;
    ROCM_CALL(unwrap(out, "out", &vOut));
    ROCM_CALL(unwrap(query, "query", &vQ));
    ROCM_CALL(unwrap(key, "key", &vK));
    ROCM_CALL(unwrap(value, "value", &vV));
    ROCM_CALL(requireDeviceContiguous(vOut, "out"));
    ROCM_CALL(requireDeviceContiguous(vQ, "query"));
    ROCM_CALL(requireDeviceContiguous(vK, "key"));
    ROCM_CALL(requireDeviceContiguous(vV, "value"));
    ROCM_CHECK(num_heads > 0 && num_kv_heads > 0 && dim > 0 && num_heads % num_kv_heads == 0 && num_heads <= INT32_MAX / 1024 && dim <= 65535,
               "num_heads %lld must be a positive multiple of num_kv_heads %lld, dim %lld positive", static_cast<long long>(num_heads),
               static_cast<long long>(num_kv_heads), static_cast<long long>(dim));
    ROCM_CHECK(actual_seq_lengths.len >= 0 && actual_seq_lengths.len <= 65535 && max_input_len >= 0 && max_input_len <= INT32_MAX,
               "batch size %lld or max_input_len %lld out of range", static_cast<long long>(actual_seq_lengths.len), static_cast<long long>(max_input_len));
    const int64_t batch = actual_seq_lengths.len;
    const int64_t rows = batch * max_input_len;
    ROCM_CHECK(vQ.ndim == 2 && vQ.shape[0] == rows && vQ.shape[1] == num_heads * dim, "query must be [batch * max_input_len, num_heads * dim] = [%lld, %lld]",
               static_cast<long long>(rows), static_cast<long long>(num_heads * dim));
    ROCM_CHECK(vOut.sameShape(vQ), "out must have the shape of query");
    ROCM_CHECK(vK.ndim == 2 && vK.shape[0] == rows && vK.shape[1] == num_kv_heads * dim && vV.sameShape(vK),
               "key and value must be [batch * max_input_len, num_kv_heads * dim] = [%lld, %lld]", static_cast<long long>(rows),
               static_cast<long long>(num_kv_heads * dim));
    ROCM_CHECK(isFloatDtype(vQ.dtype) && vK.dtype == vQ.dtype && vV.dtype == vQ.dtype && vOut.dtype == vQ.dtype,
               "query, key, value and out must share one floating dtype (query is %s)", dtypeName(vQ.dtype));
    if (rows == 0) return diopiSuccess;

    CtxArgs a;
    a.bStartLoc = nullptr;
    a.bSeqLen = nullptr;
    a.start64 = false;
    a.len64 = false;
    a.batch = static_cast<int>(batch);
    a.H = static_cast<int>(num_heads);
    a.rows = rows;
    a.tilesBound = 0;
    a.totalItems = 0;
    a.cumulative = false;
    a.uniformLen = static_cast<int>(max_input_len);
    a.causal = true;
    a.G = static_cast<int>(num_heads / num_kv_heads);
    const int D = static_cast<int>(dim);
    const double scale = 1.0 / std::sqrt(static_cast<double>(D));
    a.scaleLog2 = static_cast<float>(scale * 1.4426950408889634);
    a.lse = nullptr;
    a.lseStride = 0;
    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    const diopiError_t err = dispatchAttention<true>(ctx, stream, vOut, vQ, vK, vV, a, D, scale);
    if (err != diopiDtypeNotSupported) return err;
    setLastError("diopiPromptFlashAttention: dtype %s is not supported", dtypeName(vQ.dtype));
    return diopiDtypeNotSupported;
    ROCM_ENTRY_END
}
