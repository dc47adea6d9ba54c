// dsx_knn_f16.hip — scores of the exact KNN search with items and queries stored as fp16 (the reference's DataType::FP16:
// knn/KnnData.cpp:209-216 converts the table with kFloatToHalf, knn/KnnExactGpu.cu:108-116 converts every query batch, and
// cublasSgemmEx multiplies fp16 operands into fp32 scores).
//
// Storage is this library's own: both operands row-major with the vector's components contiguous ([item][ld] and
// [query][ld] halves, ld = dim rounded up to 64, zero filled; rows rounded up to 256, the tallest tile, zero filled), which is
// what v_mfma_f32_32x32x16_f16 wants — a lane's operand is 8 consecutive components of one row, one 128-bit read — and
// leaves the k-loop without any bounds check.  A 256-lane workgroup (2 x 2 wavefronts) owns a 128 x 128 tile of scores;
// 32 components of both operands per step are staged in LDS (double buffered, rows padded to 80 bytes so that the 128-bit
// reads of 8 lanes cover all banks once).  Products of fp16 values are exact in fp32 and the sums are fp32, as in the
// reference's GEMM.  Epilogues: plain store (first column block) or candidate lists (everything after it).
#include <algorithm>
#include "dsx_device.h"
#include "dsx_internal.h"

namespace dsx {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));

constexpr int kF16Xcds = 8;

struct KnnF16Args {
    const _Float16* A;      // queries [rows rounded up to 256][ld]
    const _Float16* B;      // items of this column range [columns rounded up to 256][ld]
    uint32_t ld;            // halves per row, a multiple of 64
    uint32_t batch, n;      // valid rows of A, valid columns (items) of this range
    uint32_t tiles_m, tiles_n;
    float* Z;               // store mode: scores [batch][ldz]
    uint32_t ldz;
    CandArgs cand;          // candidate mode
};

// MI x NI accumulator blocks of 32 x 32 per wavefront, WM x WN wavefronts per workgroup: a (32*MI*WM) x (32*NI*WN) tile, with
// as many rows and columns as half the workgroup's lanes (two 16-byte chunks per lane, operand and step).  WPE: wavefronts
// per SIMD the register budget is sized for.
template <int MI, int NI, int WM, int WN, int WPE, bool CAND>
__global__ __launch_bounds__(64 * WM * WN) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void knn_f16_kernel(KnnF16Args a)
{
    constexpr int THREADS = 64 * WM * WN;
    constexpr int BM = 32 * MI * WM, BN = 32 * NI * WN, BK = 32, PITCH = BK + 8;   // halves; 80-byte rows
    constexpr int RS = THREADS / 4;                                                // rows between a lane's two chunks
    static_assert(BM == THREADS / 2 && BN == THREADS / 2, "two chunks per lane, operand and step");
    __shared__ __attribute__((aligned(16))) _Float16 sA[2][BM][PITCH];
    __shared__ __attribute__((aligned(16))) _Float16 sB[2][BN][PITCH];

    const uint32_t total = a.tiles_m * a.tiles_n;
    uint32_t wg = blockIdx.x;
    {
        const uint32_t per_xcd = (total + kF16Xcds - 1) / kF16Xcds;
        const uint32_t xcd = wg % kF16Xcds, local = wg / kF16Xcds;
        wg = xcd * per_xcd + local;
        if (local >= per_xcd || wg >= total) return;
    }
    const uint32_t tm = wg % a.tiles_m, tn = wg / a.tiles_m;
    const uint32_t row0 = tm * BM, col0 = tn * BN;
    __builtin_amdgcn_s_setprio(3);   // k-loop first, epilogue in the issue slots that are left (as in fc_gemm_kernel)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int l32 = lane & 31, lhi = lane >> 5;

    floatx16 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    // A step of a tile is 64 bytes per row = four chunks of 16 bytes; lane t takes chunk t % 4 of rows t / 4 and t / 4 + RS of
    // both operands.  The loads of the next two steps are in flight in registers (two stages of named registers — 128-bit
    // values reached through arrays or references from inside lambdas would live in scratch memory); the step that is due
    // next is written to the LDS double buffer while the current one is multiplied.
    const int srow = tid >> 2, spart = tid & 3;
    const uint4* gA = reinterpret_cast<const uint4*>(a.A + (uint64_t)(row0 + srow) * a.ld) + spart;
    const uint4* gB = reinterpret_cast<const uint4*>(a.B + (uint64_t)(col0 + srow) * a.ld) + spart;
    const uint32_t rstep = RS * (a.ld / 8);   // chunks between a lane's two rows
    const uint32_t nk = a.ld / BK;            // a multiple of 2
#define F16_LOAD(S, KT)                                                                                                  \
    do {                                                                                                                 \
        const uint32_t o_ = min((uint32_t)(KT), nk - 1) * (BK / 8); /* past the end: the last step again, never used */  \
        S##a0 = gA[o_];                                                                                                  \
        S##a1 = gA[o_ + rstep];                                                                                          \
        S##b0 = gB[o_];                                                                                                  \
        S##b1 = gB[o_ + rstep];                                                                                          \
    } while (0)
#define F16_STORE(S, BUF)                                                         \
    do {                                                                          \
        *reinterpret_cast<uint4*>(&sA[BUF][srow][spart * 8]) = S##a0;             \
        *reinterpret_cast<uint4*>(&sA[BUF][srow + RS][spart * 8]) = S##a1;        \
        *reinterpret_cast<uint4*>(&sB[BUF][srow][spart * 8]) = S##b0;             \
        *reinterpret_cast<uint4*>(&sB[BUF][srow + RS][spart * 8]) = S##b1;        \
    } while (0)
    auto multiply = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int ks = 0; ks < BK / 16; ks++) {
            half8 av[MI], bv[NI];
#pragma unroll
            for (int i = 0; i < MI; i++) av[i] = *reinterpret_cast<const half8*>(&sA[buf][wm * 32 * MI + i * 32 + l32][ks * 16 + lhi * 8]);
#pragma unroll
            for (int j = 0; j < NI; j++) bv[j] = *reinterpret_cast<const half8*>(&sB[buf][wn * 32 * NI + j * 32 + l32][ks * 16 + lhi * 8]);
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int j = 0; j < NI; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[i], bv[j], acc[i][j], 0, 0, 0);
        }
    };

    uint32_t bound_key = 0;
    if constexpr (CAND) bound_key = candidate_bound_prefetch<MI, WM>(a.cand, row0, a.batch, tid);
    uint4 s0a0, s0a1, s0b0, s0b1, s1a0, s1a1, s1b0, s1b1;
    F16_LOAD(s0, 0);
    F16_LOAD(s1, 1);
    if constexpr (CAND) asm volatile("" ::"v"(bound_key));   // the bound's load is issued up here, not moved down to its use
    F16_STORE(s0, 0);
    __syncthreads();
    for (uint32_t kt = 0; kt < nk; kt += 2) {
        // step kt + j multiplies LDS buffer j; its stage's registers are free again and take step kt + j + 2
        F16_LOAD(s0, kt + 2);
        multiply(0);
        F16_STORE(s1, 1);
        __syncthreads();
        F16_LOAD(s1, kt + 3);
        multiply(1);
        F16_STORE(s0, 0);
        __syncthreads();
    }
#undef F16_LOAD
#undef F16_STORE

    __builtin_amdgcn_s_setprio(0);
    if constexpr (CAND) {
        static_assert(sizeof(sA) >= kCandLdsBytes<MI, WM, WN>, "the epilogue reuses the query tile's LDS");
        candidate_epilogue<MI, NI, WM, WN>(acc, reinterpret_cast<float*>(&sA[0][0][0]), a.cand, bound_key, row0, col0, a.batch, a.n, tid, wm, wn,
                                           l32, lhi);
    } else {
#pragma unroll
        for (int j = 0; j < NI; j++) {
            const uint32_t c = col0 + wn * 32 * NI + j * 32 + l32;
            if (c >= a.n) continue;
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const uint32_t r = row0 + wm * 32 * MI + i * 32 + 8 * (v / 4) + 4 * lhi + (v % 4);
                    if (r < a.batch) a.Z[(uint64_t)r * a.ldz + c] = acc[i][j][v];
                }
        }
    }
}

// Candidate mode for long column ranges: a workgroup keeps its 128 queries and sweeps a contiguous chunk of the range's item
// tiles, one after the other.  What a tile costs beyond its multiplications then shrinks to the compares:
//  * the operand stream never stops at a tile boundary — the loads of the next tile's first two steps are in flight while
//    the current tile's last steps are multiplied, so no tile waits for its first operands;
//  * the rows' bounds are read once per workgroup, not once per tile;
//  * survivors go to lists that belong to this (row, chunk) alone, a[row][chunk][seg_cap], whose fill counts live in LDS:
//    no atomic on device memory (thousands of cycles of round trip per tile in knn_f16_kernel), only a plain store.  The
//    counts are published when the sweep ends.  A (row, chunk) list that is full spills into the row's shared list, the one
//    knn_f16_kernel appends to (CandArgs), so clustered items cost time, not exactness.
// The 80-byte LDS rows of the operand tiles have 16 bytes of padding each; row r of the first query buffer keeps row r's
// fill count and bound there, so the kernel needs no LDS beyond the operand buffers and four workgroups still share a CU.
constexpr uint32_t kSweepCountStride = 64;   // seg_count is [queries][64]; chunks <= 64

struct KnnF16SweepArgs {
    const _Float16* A;      // queries [rows rounded up to 256][ld]
    const _Float16* B;      // items of this column range [columns rounded up to 256][ld]
    uint32_t ld;
    uint32_t batch, n;
    uint32_t tiles_m, tiles_n;
    uint32_t chunks, tiles_per_chunk;
    uint64_t* seg;          // [queries][chunks][seg_cap]
    uint32_t* seg_count;    // [queries][kSweepCountStride]
    uint32_t seg_cap;
    CandArgs cand;          // bounds, column offset, and the shared lists a full (row, chunk) list spills into
};

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void knn_f16_sweep_kernel(KnnF16SweepArgs a)
{
    constexpr int MI = 2, NI = 2, WN = 2, BM = 128, BN = 128, BK = 32, PITCH = BK + 8, RS = 64;
    __shared__ __attribute__((aligned(16))) _Float16 sA[2][BM][PITCH];
    __shared__ __attribute__((aligned(16))) _Float16 sB[2][BN][PITCH];

    // Workgroups that sweep the same chunk (the same item tiles, different queries) sit on the same XCD and advance at the
    // same rate: an item tile comes from HBM once and from that XCD's L2 for the others.
    const uint32_t total = a.tiles_m * a.chunks;
    uint32_t wg = blockIdx.x;
    {
        const uint32_t per_xcd = (total + kF16Xcds - 1) / kF16Xcds;
        const uint32_t xcd = wg % kF16Xcds, local = wg / kF16Xcds;
        wg = xcd * per_xcd + local;
        if (local >= per_xcd || wg >= total) return;
    }
    const uint32_t tm = wg % a.tiles_m, chunk = wg / a.tiles_m;
    const uint32_t row0 = tm * BM;
    const uint32_t t0 = chunk * a.tiles_per_chunk;
    const uint32_t t1 = min(t0 + a.tiles_per_chunk, a.tiles_n);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int l32 = lane & 31, lhi = lane >> 5;
    if (t0 >= t1) {   // more chunks than tiles: an empty list
        if (tid < BM && row0 + tid < a.batch) a.seg_count[(uint64_t)(row0 + tid) * kSweepCountStride + chunk] = 0;
        return;
    }
    // row r's state: [0] fill count of its list, [1] its bound as a float (key 0: no bound yet, everything that is a number passes)
    auto row_state = [&](int r) __attribute__((always_inline)) { return reinterpret_cast<uint32_t*>(&sA[0][r][BK]); };
    if (tid < BM) {
        float bound = __builtin_inff();   // rows beyond the batch admit nothing
        if (row0 + tid < a.batch) {
            const uint32_t key = a.cand.row_bound[row0 + tid];
            bound = key ? key_score(key) : -__builtin_inff();
        }
        row_state(tid)[0] = 0;
        row_state(tid)[1] = __float_as_uint(bound);
    }

    floatx16 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    // The operand stream: step after step of 32 components, tile after tile.  The cursor stops at the chunk's last tile (what
    // is requested beyond the end is that tile again and never used).
    const int srow = tid >> 2, spart = tid & 3;
    const uint32_t nk = a.ld / BK;   // a multiple of 2
    const uint32_t rstep = RS * (a.ld / 8);
    const uint64_t tile_step = (uint64_t)BN * (a.ld / 8);
    const uint4* gA = reinterpret_cast<const uint4*>(a.A + (uint64_t)(row0 + srow) * a.ld) + spart;
    const uint4* gB = reinterpret_cast<const uint4*>(a.B + ((uint64_t)t0 * BN + srow) * a.ld) + spart;
    uint32_t cur_kt = 0, cur_t = t0;
#define F16_LOAD(S)                                \
    do {                                           \
        const uint32_t o_ = cur_kt * (BK / 8);     \
        S##a0 = gA[o_];                            \
        S##a1 = gA[o_ + rstep];                    \
        S##b0 = gB[o_];                            \
        S##b1 = gB[o_ + rstep];                    \
        if (++cur_kt == nk) {                      \
            cur_kt = 0;                            \
            if (cur_t + 1 < t1) {                  \
                cur_t++;                           \
                gB += tile_step;                   \
            }                                      \
        }                                          \
    } while (0)
#define F16_STORE(S, BUF)                                                         \
    do {                                                                          \
        *reinterpret_cast<uint4*>(&sA[BUF][srow][spart * 8]) = S##a0;             \
        *reinterpret_cast<uint4*>(&sA[BUF][srow + RS][spart * 8]) = S##a1;        \
        *reinterpret_cast<uint4*>(&sB[BUF][srow][spart * 8]) = S##b0;             \
        *reinterpret_cast<uint4*>(&sB[BUF][srow + RS][spart * 8]) = S##b1;        \
    } while (0)
    auto multiply = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int ks = 0; ks < BK / 16; ks++) {
            half8 av[MI], bv[NI];
#pragma unroll
            for (int i = 0; i < MI; i++) av[i] = *reinterpret_cast<const half8*>(&sA[buf][wm * 32 * MI + i * 32 + l32][ks * 16 + lhi * 8]);
#pragma unroll
            for (int j = 0; j < NI; j++) bv[j] = *reinterpret_cast<const half8*>(&sB[buf][wn * 32 * NI + j * 32 + l32][ks * 16 + lhi * 8]);
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int j = 0; j < NI; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[i], bv[j], acc[i][j], 0, 0, 0);
        }
    };

    uint4 s0a0, s0a1, s0b0, s0b1, s1a0, s1a1, s1b0, s1b1;
    F16_LOAD(s0);
    F16_LOAD(s1);
    F16_STORE(s0, 0);
    __syncthreads();   // also publishes the rows' state
    for (uint32_t t = t0; t < t1; t++) {
        __builtin_amdgcn_s_setprio(3);   // multiplying wavefronts first, comparing ones in the issue slots that are left
        for (uint32_t kt = 0; kt < nk; kt += 2) {
            F16_LOAD(s0);
            multiply(0);
            F16_STORE(s1, 1);
            __syncthreads();
            F16_LOAD(s1);
            multiply(1);
            F16_STORE(s0, 0);   // after a tile's last step: the next tile's first
            __syncthreads();
        }
        __builtin_amdgcn_s_setprio(0);
        // The tile against the rows' bounds: one compare per score; a 32 x 32 block without survivors costs nothing else.
        const uint32_t colbase = t * BN + wn * 32 * NI;
#pragma unroll
        for (int i = 0; i < MI; i++) {
            float bf[16];
#pragma unroll
            for (int v = 0; v < 16; v++) bf[v] = __uint_as_float(row_state(wm * 32 * MI + i * 32 + 8 * (v / 4) + 4 * lhi + (v % 4))[1]);
#pragma unroll
            for (int j = 0; j < NI; j++) {
                uint64_t any = 0;
#pragma unroll
                for (int v = 0; v < 16; v++) any |= __builtin_amdgcn_ballot_w64(acc[i][j][v] >= bf[v]);
                if (any != 0) {
                    const uint32_t col = colbase + j * 32 + l32;
                    const bool col_ok = col < a.n;   // columns beyond the range hold sums over zero padding
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        float x = acc[i][j][v];
                        asm volatile("" : "+v"(x));
                        const bool pass = x >= bf[v] && col_ok;
                        if (__builtin_amdgcn_ballot_w64(pass) == 0) continue;
                        if (pass) {
                            // (the row is made opaque so that the list addresses of all 64 registers are worked out here, where one
                            // is needed, and not kept in registers across the sweep)
                            uint32_t rl = wm * 32 * MI + i * 32 + 8 * (v / 4) + 4 * lhi + (v % 4);
                            asm volatile("" : "+v"(rl));
                            const uint32_t r = row0 + rl;
                            const uint64_t word = ((uint64_t)score_key(x) << 32) | (uint32_t)~(a.cand.col_offset + col);
                            const uint32_t pos = atomicAdd(&row_state(rl)[0], 1u);
                            if (pos < a.seg_cap) {
                                a.seg[((uint64_t)r * a.chunks + chunk) * a.seg_cap + pos] = word;
                            } else {   // this (row, chunk) list is full: the row's shared list
                                const uint32_t p2 = atomicAdd(&a.cand.cand_count[r], 1u);
                                if (p2 < a.cand.cand_cap) a.cand.cand[(uint64_t)r * a.cand.cand_cap + p2] = word;
                                else *a.cand.overflow = 1u;
                            }
                        }
                    }
                }
#pragma unroll
                for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;
            }
        }
    }
#undef F16_LOAD
#undef F16_STORE
    __syncthreads();
    if (tid < BM && row0 + tid < a.batch)
        a.seg_count[(uint64_t)(row0 + tid) * kSweepCountStride + chunk] = min(row_state(tid)[0], a.seg_cap);
}

// Candidate mode for long column ranges when the vectors have at most 256 components: the queries live in registers.
// A wavefront keeps the operand fragments of its 64 queries for every k-step (KS * 8 registers), so the only operand that
// moves during the sweep is the item: 64 items per stage, whole rows, staged in LDS once per workgroup of eight wavefronts
// (512 queries) and read from there as the other MFMA operand — one 128-bit LDS read feeds two multiplications, where
// knn_f16_sweep_kernel needs one read each, and a CU pulls in a quarter of the item bytes per multiplication.  The items are
// the row operand, so a lane's sixteen results of a multiplication are sixteen items of ONE query: its bound is one register
// and a few maxima and one compare are all a block without survivors costs.  The lists have the layout knn_f16_sweep_kernel
// fills, with two lists per (query, chunk) — one for each of the two lanes that hold items of that query — whose fill counts
// are registers; a full list spills into the query's shared list.  One workgroup per CU: two wavefronts per SIMD with 256
// registers each.
constexpr int kWideStageItems = 128;
template <int KS>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void knn_f16_wide_kernel(KnnF16SweepArgs a)
{
    constexpr int BQ = 512, BI = kWideStageItems, LD = KS * 16, PITCH = LD + 8, THREADS = 512;
    constexpr int PIECES = BI * (LD / 8) / THREADS;   // 16-byte pieces of a stage per lane
    static_assert(BI * (LD / 8) % THREADS == 0, "a stage is a whole number of 16-byte pieces per lane");
    extern __shared__ __attribute__((aligned(16))) unsigned char wide_lds[];
    typedef _Float16 (*StagePtr)[BI][PITCH];
    StagePtr sI = reinterpret_cast<StagePtr>(wide_lds);   // two stages of items

    // Workgroups that sweep the same chunk sit on the same XCD: an item stage comes from HBM once and from that XCD's L2 for
    // the others.
    const uint32_t total = a.tiles_m * a.chunks;
    uint32_t wg = blockIdx.x;
    {
        const uint32_t per_xcd = (total + kF16Xcds - 1) / kF16Xcds;
        const uint32_t xcd = wg % kF16Xcds, local = wg / kF16Xcds;
        wg = xcd * per_xcd + local;
        if (local >= per_xcd || wg >= total) return;
    }
    const uint32_t tm = wg % a.tiles_m, chunk = wg / a.tiles_m;
    const uint32_t row0 = tm * BQ;
    const uint32_t s0 = chunk * a.tiles_per_chunk;                 // stages of BI items
    const uint32_t s1 = min(s0 + a.tiles_per_chunk, a.tiles_n);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lhi = lane >> 5;
    if (s0 >= s1) {   // more chunks than stages: two empty lists per query
        if (row0 + tid < a.batch) {
            a.seg_count[(uint64_t)(row0 + tid) * kSweepCountStride + 2 * chunk] = 0;
            a.seg_count[(uint64_t)(row0 + tid) * kSweepCountStride + 2 * chunk + 1] = 0;
        }
        return;
    }

    // this lane's two queries: operand fragments for all k-steps, and their bounds (key 0: no bound yet, every number passes)
    const uint32_t rows_stored = (a.batch + 255) / 256 * 256;   // rows the query array holds (zero filled beyond the batch)
    uint32_t q[2];
    uint64_t* my_seg[2];   // list (query, 2 * chunk + lhi) of seg_cap words
    half8 bq[2][KS];
    float bound[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        q[h] = row0 + wave * 64 + h * 32 + l32;
        my_seg[h] = a.seg + ((uint64_t)q[h] * (2 * a.chunks) + 2 * chunk + lhi) * a.seg_cap;
        const _Float16* qp = a.A + (uint64_t)min(q[h], rows_stored - 1) * LD + lhi * 8;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) bq[h][ks] = *reinterpret_cast<const half8*>(qp + ks * 16);
        bound[h] = __builtin_inff();   // queries beyond the batch admit nothing
        if (q[h] < a.batch) {
            const uint32_t key = a.cand.row_bound[q[h]];
            bound[h] = key ? key_score(key) : -__builtin_inff();
        }
    }

    // A stage is BI whole rows: one contiguous piece of the table.
    const uint4* gI = reinterpret_cast<const uint4*>(a.B + (uint64_t)s0 * BI * LD) + tid;
    // (named registers, not an array: an array that a conditional load fills ends up in scratch memory)
    uint4 st0 = {}, st1 = {}, st2 = {}, st3 = {}, st4 = {}, st5 = {}, st6 = {}, st7 = {};
    static_assert(PIECES >= 1 && PIECES <= 8, "one to eight pieces per lane");
    auto load_stage = [&]() __attribute__((always_inline)) {
        st0 = gI[0];
        if constexpr (PIECES > 1) st1 = gI[THREADS];
        if constexpr (PIECES > 2) st2 = gI[2 * THREADS];
        if constexpr (PIECES > 3) st3 = gI[3 * THREADS];
        if constexpr (PIECES > 4) st4 = gI[4 * THREADS];
        if constexpr (PIECES > 5) st5 = gI[5 * THREADS];
        if constexpr (PIECES > 6) st6 = gI[6 * THREADS];
        if constexpr (PIECES > 7) st7 = gI[7 * THREADS];
        gI += BI * (LD / 8);
    };
    auto store_piece = [&](int buf, int j, const uint4& v) __attribute__((always_inline)) {
        const int p = tid + j * THREADS;
        *reinterpret_cast<uint4*>(&sI[buf][p / (LD / 8)][(p % (LD / 8)) * 8]) = v;
    };
    auto store_stage = [&](int buf) __attribute__((always_inline)) {
        store_piece(buf, 0, st0);
        if constexpr (PIECES > 1) store_piece(buf, 1, st1);
        if constexpr (PIECES > 2) store_piece(buf, 2, st2);
        if constexpr (PIECES > 3) store_piece(buf, 3, st3);
        if constexpr (PIECES > 4) store_piece(buf, 4, st4);
        if constexpr (PIECES > 5) store_piece(buf, 5, st5);
        if constexpr (PIECES > 6) store_piece(buf, 6, st6);
        if constexpr (PIECES > 7) store_piece(buf, 7, st7);
    };
    // The 32 x 32 scores of one query block against one item block.  A lane holds sixteen items of one query, and the two
    // lanes that share a query (rows 4 * lhi + ...) each own a list of their own — (query, 2 * chunk + lhi) — so a
    // survivor costs a store and a register increment, no atomic.  The largest of the sixteen first (three-way maxima by
    // groups of four), then only the groups and scores that reach the bound.
    uint32_t fill[2] = {0, 0};
    auto compare = [&](const floatx16& acc, int h, uint32_t item0) __attribute__((always_inline)) {
        float gm[4];
#pragma unroll
        for (int g = 0; g < 4; g++) gm[g] = fmaxf(fmaxf(fmaxf(acc[4 * g], acc[4 * g + 1]), acc[4 * g + 2]), acc[4 * g + 3]);
        const float top = fmaxf(fmaxf(fmaxf(gm[0], gm[1]), gm[2]), gm[3]);
        if (__builtin_amdgcn_ballot_w64(top >= bound[h]) == 0) return;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            if (__builtin_amdgcn_ballot_w64(gm[g] >= bound[h]) == 0) continue;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float x = acc[4 * g + e];
                asm volatile("" : "+v"(x));
                const uint32_t col = item0 + 8 * g + e;
                if (x >= bound[h] && col < a.n) {   // (items beyond the range are zero padding)
                    const uint64_t word = ((uint64_t)score_key(x) << 32) | (uint32_t)~(a.cand.col_offset + col);
                    if (fill[h] < a.seg_cap) {
                        my_seg[h][fill[h]] = word;
                    } else {   // this list is full: the query's shared list
                        const uint32_t p2 = atomicAdd(&a.cand.cand_count[q[h]], 1u);
                        if (p2 < a.cand.cand_cap) a.cand.cand[(uint64_t)q[h] * a.cand.cand_cap + p2] = word;
                        else *a.cand.overflow = 1u;
                    }
                    fill[h]++;
                }
            }
        }
    };

    load_stage();
    store_stage(0);
    __syncthreads();
    for (uint32_t s = s0; s < s1; s++) {
        const int buf = (int)((s - s0) & 1u);
        const bool more = s + 1 < s1;
        if (more) load_stage();
        // The item fragment of step ks + AHEAD is requested before step ks multiplies, so that the LDS latency is paid once per
        // item block and not once per step.
        constexpr int AHEAD = (KS < 6) ? KS : 6, RING = 8;
#pragma unroll 1
        for (int sub = 0; sub < BI / 32; sub++) {
            const _Float16* ip = &sI[buf][sub * 32 + l32][lhi * 8];
            half8 av[RING];
#pragma unroll
            for (int t = 0; t < AHEAD; t++) av[t % RING] = *reinterpret_cast<const half8*>(ip + t * 16);
            __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);   // the first AHEAD reads,
            floatx16 acc0, acc1;
#pragma unroll
            for (int v = 0; v < 16; v++) acc0[v] = acc1[v] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                if (ks + AHEAD < KS) av[(ks + AHEAD) % RING] = *reinterpret_cast<const half8*>(ip + (ks + AHEAD) * 16);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[ks % RING], bq[0][ks], acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[ks % RING], bq[1][ks], acc1, 0, 0, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);                        // then two multiplications
                if (ks + AHEAD < KS) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // and one more read, in turn
            }
            const uint32_t item0 = s * BI + sub * 32 + 4 * lhi;
            compare(acc0, 0, item0);
            compare(acc1, 1, item0);
        }
        if (more) store_stage(buf ^ 1);
        __syncthreads();
    }
#pragma unroll
    for (int h = 0; h < 2; h++)
        if (q[h] < a.batch) a.seg_count[(uint64_t)q[h] * kSweepCountStride + 2 * chunk + lhi] = min(fill[h], a.seg_cap);
}

template <int KS> static int launch_wide(const KnnF16SweepArgs& a, uint32_t grid)
{
    constexpr size_t lds = 2 * kWideStageItems * (KS * 16 + 8) * sizeof(_Float16);
    static bool sized[64] = {};   // per device: the kernel's LDS limit is raised once
    const int dev = ctx().device;
    if (dev < 0 || dev >= 64 || !sized[dev]) {
        DSX_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&knn_f16_wide_kernel<KS>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        if (dev >= 0 && dev < 64) sized[dev] = true;
    }
    hipLaunchKernelGGL((knn_f16_wide_kernel<KS>), dim3(grid), dim3(512), lds, ctx().stream, a);
    DSX_LAUNCH_CHECK("knn_f16_wide_kernel");
    return DSX_OK;
}

// fp32 -> fp16, round to nearest even (__float2half), into the padded row-major layout.  src is either column-major
// (items: src[d * src_ld + row]) or row-major (queries: src[row * src_ld + d]); rows >= rows_valid and components >= dim
// become zero.  One lane per 8 output halves.
template <bool COLMAJOR>
__global__ __launch_bounds__(256) void knn_to_f16_kernel(const float* src, uint64_t src_ld, uint32_t rows_valid, uint32_t dim, _Float16* dst,
                                                         uint32_t rows_out, uint32_t ld)
{
    const uint64_t chunk = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    const uint32_t per_row = ld / 8;
    uint32_t row, part;
    if constexpr (COLMAJOR) {
        // consecutive lanes take consecutive rows of one 8-component group: the reads of a component are then contiguous
        const uint64_t rows64 = rows_out;
        part = (uint32_t)(chunk / rows64);
        row = (uint32_t)(chunk % rows64);
        if (part >= per_row) return;
    } else {
        row = (uint32_t)(chunk / per_row);
        part = (uint32_t)(chunk % per_row);
        if (row >= rows_out) return;
    }
    half8 h;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const uint32_t d = part * 8 + e;
        float x = 0.0f;
        if (row < rows_valid && d < dim) x = COLMAJOR ? src[(uint64_t)d * src_ld + row] : src[(uint64_t)row * src_ld + d];
        h[e] = (_Float16)x;
    }
    *reinterpret_cast<half8*>(dst + (uint64_t)row * ld + part * 8) = h;
}

uint32_t knn_f16_ld(uint32_t dim) { return (dim + 63) / 64 * 64; }   // two pipeline steps of 32 components
uint64_t knn_f16_rows(uint64_t rows) { return (rows + 255) / 256 * 256; }   // the tallest tile

int knn_to_f16(const float* src, bool colmajor, uint64_t src_ld, uint32_t rows_valid, uint32_t dim, void* dst, uint32_t rows_out)
{
    const uint32_t ld = knn_f16_ld(dim);
    const uint64_t chunks = (uint64_t)rows_out * (ld / 8);
    const uint32_t grid = (uint32_t)((chunks + 255) / 256);
    if (colmajor)
        hipLaunchKernelGGL((knn_to_f16_kernel<true>), dim3(grid), dim3(256), 0, ctx().stream, src, src_ld, rows_valid, dim, (_Float16*)dst, rows_out, ld);
    else
        hipLaunchKernelGGL((knn_to_f16_kernel<false>), dim3(grid), dim3(256), 0, ctx().stream, src, src_ld, rows_valid, dim, (_Float16*)dst, rows_out, ld);
    DSX_LAUNCH_CHECK("knn_to_f16_kernel");
    return DSX_OK;
}

template <int MI, int NI, int WM, int WN, int WPE> static void launch_f16(KnnF16Args& a, const CandArgs* cand)
{
    constexpr int BM = 32 * MI * WM, BN = 32 * NI * WN;
    a.tiles_m = (a.batch + BM - 1) / BM;
    a.tiles_n = (a.n + BN - 1) / BN;
    const uint32_t total = a.tiles_m * a.tiles_n;
    const uint32_t grid = ((total + kF16Xcds - 1) / kF16Xcds) * kF16Xcds;
    if (cand) {
        a.cand = *cand;
        hipLaunchKernelGGL((knn_f16_kernel<MI, NI, WM, WN, WPE, true>), dim3(grid), dim3(64 * WM * WN), 0, ctx().stream, a);
    } else {
        hipLaunchKernelGGL((knn_f16_kernel<MI, NI, WM, WN, WPE, false>), dim3(grid), dim3(64 * WM * WN), 0, ctx().stream, a);
    }
}

// Scores of `batch` queries against `n` items starting at items16 (both in the padded fp16 layout): stored into Z[batch][ldz]
// when cand == NULL, compared with the queries' bounds otherwise.
int knn_f16_scores_run(const void* queries16, const void* items16, uint32_t ld, uint32_t batch, uint32_t n, float* Z, uint32_t ldz,
                       const CandArgs* cand)
{
    KnnF16Args a{};
    a.A = (const _Float16*)queries16;
    a.B = (const _Float16*)items16;
    a.ld = ld;
    a.batch = batch;
    a.n = n;
    a.Z = Z;
    a.ldz = ldz;
    // 128 x 128 tiles, four workgroups per CU (their 40 KiB of LDS each fill the CU's 160 KiB).  Measured against it on config 5:
    // 256 x 256 tiles with eight wavefronts (6.6 ms vs 6.0), three workgroups per CU (6.3 ms).
    launch_f16<2, 2, 2, 2, 4>(a, cand);
    DSX_LAUNCH_CHECK("knn_f16_kernel");
    return DSX_OK;
}

// Candidate mode of a column range of n items for `batch` queries.  mode 0: one workgroup per tile (knn_f16_kernel); 1: a
// sweep when it has workgroups for (half of) the CUs and enough items per chunk — knn_f16_wide_kernel for vectors of at most 256
// components, knn_f16_sweep_kernel otherwise; 2: knn_f16_sweep_kernel whenever every chunk gets a tile, 3: knn_f16_wide_kernel
// whenever every chunk gets a stage (tests at small sizes).  *chunks_used: the chunks of the sweep, 0 when the range went
// through knn_f16_kernel and only the shared lists were appended to.
int knn_f16_candidates_run(const void* queries16, const void* items16, uint32_t ld, uint32_t batch, uint32_t n, const CandArgs& cand,
                           uint64_t* seg, uint32_t* seg_count, uint32_t seg_words, int mode, uint32_t* chunks_used)
{
    *chunks_used = 0;
    const uint32_t cus = (uint32_t)ctx().num_cus;
    KnnF16SweepArgs a{};
    a.A = (const _Float16*)queries16;
    a.B = (const _Float16*)items16;
    a.ld = ld;
    a.batch = batch;
    a.n = n;
    a.seg = seg;
    a.seg_count = seg_count;
    a.cand = cand;
    if (seg && seg_count && ld <= 256 && (mode == 1 || mode == 3)) {
        // queries in registers: 512 per workgroup, stages of 64 items, one workgroup per CU
        const uint32_t tiles_q = (batch + 511) / 512, stages = (n + kWideStageItems - 1) / kWideStageItems;
        const uint32_t chunks = std::min<uint32_t>(kSweepCountStride / 2, (cus + tiles_q - 1) / tiles_q);   // two lists per (query, chunk)
        if (mode == 3 ? stages >= chunks : (2 * tiles_q * chunks >= cus && stages >= 8 * chunks)) {
            a.tiles_m = tiles_q;
            a.tiles_n = stages;
            a.chunks = chunks;
            a.tiles_per_chunk = (stages + chunks - 1) / chunks;
            a.seg_cap = seg_words / (2 * chunks);
            const uint32_t total = tiles_q * chunks;
            const uint32_t grid = ((total + kF16Xcds - 1) / kF16Xcds) * kF16Xcds;
            *chunks_used = 2 * chunks;
            switch (ld) {
            case 64: return launch_wide<4>(a, grid);
            case 128: return launch_wide<8>(a, grid);
            case 192: return launch_wide<12>(a, grid);
            default: return launch_wide<16>(a, grid);
            }
        }
    }
    const uint32_t tiles_m = (batch + 127) / 128, tiles_n = (n + 127) / 128;
    const uint32_t chunks = std::min<uint32_t>(kSweepCountStride, (4 * cus + tiles_m - 1) / tiles_m);   // every CU four times over
    const bool sweep = seg && seg_count && (mode == 2 || mode == 3 ? tiles_n >= chunks : (mode == 1 && tiles_m * chunks >= 2 * cus && tiles_n >= 4 * chunks));
    if (!sweep) return knn_f16_scores_run(queries16, items16, ld, batch, n, nullptr, 0, &cand);
    a.tiles_m = tiles_m;
    a.tiles_n = tiles_n;
    a.chunks = chunks;
    a.tiles_per_chunk = (tiles_n + chunks - 1) / chunks;
    a.seg_cap = seg_words / chunks;
    const uint32_t total = a.tiles_m * a.chunks;
    const uint32_t grid = ((total + kF16Xcds - 1) / kF16Xcds) * kF16Xcds;
    hipLaunchKernelGGL(knn_f16_sweep_kernel, dim3(grid), dim3(256), 0, ctx().stream, a);
    DSX_LAUNCH_CHECK("knn_f16_sweep_kernel");
    *chunks_used = chunks;
    return DSX_OK;
}

}  // namespace dsx
