// dsx_fc.hip — dense forward of a fully connected layer: fp32 MFMA GEMM with bias, accumulate and activation fused in the
// epilogue, plus the stand-alone activation kernels.
//
// GEMM: Z[B x n] = act(acc? Z : 0 + bias + X[B x k] . W[k x n]).  A 256-lane workgroup (2 x 2 wavefronts) owns a
// (64*MI) x (64*NI) tile of Z; each wavefront keeps MI x NI accumulators of v_mfma_f32_32x32x2_f32 (32 x 32 fp32 each) in
// registers.  X and W tiles of 16 k-steps are staged k-major in LDS (double buffered, one barrier per step) so that the
// 64 lanes of an MFMA operand read 2 x 32 consecutive floats.  Workgroup ids are remapped so that the workgroups that land
// on one XCD (id mod 8) sweep all row tiles of a few column tiles: a W tile is then fetched by one L2 only.
#include <type_traits>
#include "dsx_device.h"
#include "dsx_internal.h"

namespace dsx {

constexpr int kFcThreads = 256;
constexpr int kXcds = 8;

struct FcArgs {
    const float* X;
    const float* W;
    const float* bias;
    float* Z;
    uint32_t ldx, ldw, ldz;
    uint32_t batch, k, n;
    uint32_t tiles_m, tiles_n;
    int accumulate;
    uint32_t act;
    int fast32;          // every byte offset into X and W fits 32 bits (interior tiles then take the lean load path)
    float* seg_max;      // optional: [batch][nseg] maxima of the activated outputs over 64-column segments
    uint32_t nseg;
    float slope, alpha, lambda;
    CandArgs cand;       // candidate mode (template flag CAND): Z is not written, see candidate_epilogue
    // fc_small_kernel only: also write Z as bf16 planes (the next layer's operand in the split-products mode), as fc_split_kernel would
    uint4* out_planes;
    uint32_t out_rows_padded, out_kblocks;
};

// Epilogue shared by the GEMM kernels: bias, accumulate, activation, store, and on request the maxima of 64-column segments.
// (row_w, col_w): origin of this wavefront's (32 MI) x (32 NI) part of Z.  sT: 512 floats of LDS that belong to this
// wavefront alone (only touched when a.seg_max is set).
template <int MI, int NI, int ACT>
__device__ __forceinline__ void fc_epilogue(floatx16 (&acc)[MI][NI], const FcArgs& a, uint32_t row_w, uint32_t col_w, int lane, float* sT)
{
    const int l32 = lane & 31, lhi = lane >> 5;
    // Epilogue: accumulator register v of lane l holds row 8*(v/4) + 4*(l/32) + v%4, column l%32 of its 32x32 block.
    // With seg_max set (128 x 128 tiles only), every wavefront also reduces the 64 columns it owns to one maximum per row:
    // a later top-K can then skip the column segments that cannot hold a result.
    constexpr bool kCanSegMax = (MI == 2 && NI == 2);
    const bool want_max = kCanSegMax && a.seg_max != nullptr;
    float smax[kCanSegMax ? 32 : 1];
    if constexpr (kCanSegMax) {
#pragma unroll
        for (int q = 0; q < 32; q++) smax[q] = -__builtin_inff();
    }
    // Interior tiles: every store is "wave-uniform row base + this lane's constant 32-bit byte offset" (scalar address
    // arithmetic only), the accumulate case is a branch around the whole loop and not one per element (so the 64 outputs of
    // a wavefront are independent instructions the scheduler can interleave), and the sigmoid folds the bias and the
    // exponent's scale into one multiply-add.  Vector instructions here are matrix-core time lost, see above.
    const uint32_t row_u = __builtin_amdgcn_readfirstlane(row_w), col_u = __builtin_amdgcn_readfirstlane(col_w);
    const bool full_tile = (row_u + 32 * MI <= a.batch) && (col_u + 32 * NI <= a.n) && a.ldz < (1u << 27);
    if (full_tile) {
        const uint32_t lane_off = (4u * lhi * a.ldz + l32) * 4u;
        auto interior = [&](auto accumulate_tag) __attribute__((always_inline)) {
            constexpr bool ACCUM = decltype(accumulate_tag)::value;
            constexpr float kNegLog2e = -1.4426950408889634f;
            // (row index outermost, the column blocks innermost: an accumulator register is dead as soon as its output is
            // stored and folded into the row's maximum, so the maxima need no registers of their own on top of the tile)
            float bias[NI];
#pragma unroll
            for (int j = 0; j < NI; j++) {
                bias[j] = a.bias ? a.bias[col_u + j * 32 + l32] : 0.0f;
                if constexpr (ACT == DSX_ACT_SIGMOID && !ACCUM) bias[j] *= kNegLog2e;
            }
#pragma unroll
            for (int i = 0; i < MI; i++) {
                char* base = reinterpret_cast<char*>(a.Z) + ((uint64_t)(row_u + i * 32) * a.ldz + col_u) * 4;
#pragma unroll
                for (int v = 0; v < 16; v++) {
#pragma unroll
                    for (int j = 0; j < NI; j++) {
                        float* dst = reinterpret_cast<float*>(base + (uint64_t)(8 * (v / 4) + (v % 4)) * a.ldz * 4 + j * 128 + lane_off);
                        float y;
                        if constexpr (ACT == DSX_ACT_SIGMOID && !ACCUM) {
                            y = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(fmaf(acc[i][j][v], kNegLog2e, bias[j])));
                        } else {
                            float x = acc[i][j][v] + bias[j];
                            if constexpr (ACCUM) x += *dst;
                            y = activate<ACT>(x, a.slope, a.alpha, a.lambda);
                        }
                        *dst = y;
                        if constexpr (kCanSegMax) smax[i * 16 + v] = (j == 0) ? y : fmaxf(smax[i * 16 + v], y);
                    }
                }
            }
        };
        if (a.accumulate) interior(std::true_type{});
        else interior(std::false_type{});
    } else {
#pragma unroll
        for (int j = 0; j < NI; j++) {
            const uint32_t c = col_u + j * 32 + l32;
            if (c >= a.n) continue;
            const float bias = a.bias ? a.bias[c] : 0.0f;
#pragma unroll
            for (int i = 0; i < MI; i++) {
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const uint32_t r = row_u + i * 32 + 8 * (v / 4) + 4 * lhi + (v % 4);
                    if (r < a.batch) {
                        float* dst = a.Z + (uint64_t)r * a.ldz + c;
                        float x = acc[i][j][v] + bias;
                        if (a.accumulate) x += *dst;
                        const float y = activate<ACT>(x, a.slope, a.alpha, a.lambda);
                        *dst = y;
                        if constexpr (kCanSegMax) smax[i * 16 + v] = fmaxf(smax[i * 16 + v], y);
                    }
                }
            }
        }
    }
    if constexpr (kCanSegMax) {
        if (want_max) {
            // Each lane holds 32 row maxima over its own column; what is wanted is, per row, the maximum over the 32 lanes of a
            // half wave.  Transposed through LDS, eight row indices at a time (2 KiB per wavefront): LDS instructions do not
            // compete with the matrix cores the way a cross-lane reduction in vector registers would.  Lane L reads an eighth
            // of the 32 values of result e = L / 4 (row index 8c + e % 8, lane half e / 8), rotated by e so that the lanes of
            // a quad and the 16 results spread over all banks; the four partial maxima meet through two lane exchanges.
            const int e = lane >> 2, part = lane & 3;
            const uint32_t seg = col_u / 64;
#pragma unroll
            for (int c = 0; c < 4; c++) {
#pragma unroll
                for (int q = 0; q < 8; q++) sT[q * 64 + lane] = smax[8 * c + q];
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                float m = -__builtin_inff();
#pragma unroll
                for (int u = 0; u < 8; u++) m = fmaxf(m, sT[(e & 7) * 64 + (e >> 3) * 32 + part * 8 + ((u + e) & 7)]);
                m = fmaxf(m, __shfl_xor(m, 1));
                m = fmaxf(m, __shfl_xor(m, 2));
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();   // the next round overwrites what was just read
                const int q = 8 * c + (e & 7), i = q >> 4, v = q & 15;
                const uint32_t r = row_u + i * 32 + 8 * (v >> 2) + 4 * (e >> 3) + (v & 3);
                if (part == 0 && r < a.batch && seg < a.nseg) a.seg_max[(uint64_t)r * a.nseg + seg] = m;
            }
        }
    }
}

// MI, NI: 32x32 MFMA blocks per wavefront in M and N.  XV / WV: vector width (floats) of the global loads of X / W.
// TRANS: W is stored [n][k].
// CAND: 0 = the result is stored (epilogue above); 1 = candidate mode, scores compared with score bounds (exact KNN);
// 2 = candidate mode of a layer: the accumulators start from the bias, pre-activation sums are compared with bounds derived
// from activated scores, and the survivors are activated (candidate_epilogue, PRE).  That mode needs a few registers more than
// 128 (its bounds and the bias beside the two-steps-per-trip loop): it is built for three workgroups per CU instead of spilling
// at four (config 4, 4,096 x 512 x 1,000,000: 32.2 ms per step against 33.1 with one step per trip and four workgroups).
template <int MI, int NI, int BK, int XV, int WV, bool TRANS, int ACT, int CAND = 0>
__global__ __launch_bounds__(kFcThreads, (MI * NI >= 4) ? (CAND == 2 ? 3 : 4) : 2) void fc_gemm_kernel(FcArgs a)
{
    constexpr int BM = 64 * MI, BN = 64 * NI;
    // (X tiles 32 deep: the eight lanes that hold one row's 16-byte pieces store rows of sA that are 4 * LDA floats apart; with
    // LDA = BM + 4 they fall on two LDS banks — a third of the LDS cycles of a 4,096 x 1,024 x 1,024 layer were bank conflicts —,
    // with an odd LDA on eight)
    constexpr int LDA = BM + ((BK == 32 && XV == 4) ? 1 : 4), LDB = BN + 4;
    constexpr int A_ELEMS = BM * BK / kFcThreads;   // floats of the X tile per lane
    constexpr int B_ELEMS = BN * BK / kFcThreads;
    __shared__ float sA[2][BK][LDA];
    __shared__ float sB[2][BK][LDB];

    // XCD-aware tile order
    const uint32_t total = a.tiles_m * a.tiles_n;
    uint32_t wg = blockIdx.x;
    {
        const uint32_t per_xcd = (total + kXcds - 1) / kXcds;
        const uint32_t xcd = wg % kXcds, local = wg / kXcds;
        wg = xcd * per_xcd + local;
        if (local >= per_xcd || wg >= total) return;
    }
    // Column tiles are taken from the last to the first: a partial last tile (bounds-checked loads and stores, several times
    // slower than an interior tile) then starts with the first round of workgroups instead of ending the launch alone.
    const uint32_t tm = wg % a.tiles_m, tn = a.tiles_n - 1 - wg / a.tiles_m;
    const uint32_t row0 = tm * BM, col0 = tn * BN;

    // Wavefronts in the k-loop go first, wavefronts in the epilogue take the issue slots that are left: the matrix cores then
    // idle less while a workgroup activates and stores its tile (measured 1.5 % on a 1024 x 128 x 27,278 layer).
    __builtin_amdgcn_s_setprio(1);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lhi = lane >> 5;

    floatx16 acc[MI][NI];
#pragma unroll
    for (int j = 0; j < NI; j++) {
        float start = 0.0f;
        if constexpr (CAND == 2) {   // every register of a lane belongs to column l32 of its block: the sums start from the bias
            const uint32_t c = col0 + wn * 32 * NI + j * 32 + l32;
            if (a.bias && c < a.n) start = a.bias[c];
        }
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = start;
    }

    float ra[A_ELEMS], rb[B_ELEMS];
    uint32_t bound_key = 0;
    if constexpr (CAND) bound_key = candidate_bound_prefetch<MI>(a.cand, row0, a.batch, tid);

    // X tile: element (i, kk) of the tile is X[row0 + i][k0 + kk]; lanes walk k fastest.
    auto load_a = [&](uint32_t k0) {
        if constexpr (XV == 4) {
#pragma unroll
            for (int p = 0; p < A_ELEMS / 4; p++) {
                const int idx = tid + p * kFcThreads;
                const int i = idx / (BK / 4), k4 = (idx % (BK / 4)) * 4;
                const uint32_t r = row0 + i, kk = k0 + k4;
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (r < a.batch) {
                    const float* src = a.X + (uint64_t)r * a.ldx + kk;
                    if (kk + 4 <= a.k) {
                        v = *reinterpret_cast<const float4*>(src);
                    } else {
                        if (kk < a.k) v.x = src[0];
                        if (kk + 1 < a.k) v.y = src[1];
                        if (kk + 2 < a.k) v.z = src[2];
                    }
                }
                ra[p * 4 + 0] = v.x; ra[p * 4 + 1] = v.y; ra[p * 4 + 2] = v.z; ra[p * 4 + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int p = 0; p < A_ELEMS; p++) {
                const int idx = tid + p * kFcThreads;
                const int i = idx / BK, kk = idx % BK;
                const uint32_t r = row0 + i;
                ra[p] = (r < a.batch && k0 + kk < a.k) ? a.X[(uint64_t)r * a.ldx + k0 + kk] : 0.0f;
            }
        }
    };
    auto store_a = [&](int buf) {
        if constexpr (XV == 4) {
#pragma unroll
            for (int p = 0; p < A_ELEMS / 4; p++) {
                const int idx = tid + p * kFcThreads;
                const int i = idx / (BK / 4), k4 = (idx % (BK / 4)) * 4;
#pragma unroll
                for (int c = 0; c < 4; c++) sA[buf][k4 + c][i] = ra[p * 4 + c];
            }
        } else {
#pragma unroll
            for (int p = 0; p < A_ELEMS; p++) {
                const int idx = tid + p * kFcThreads;
                sA[buf][idx % BK][idx / BK] = ra[p];
            }
        }
    };
    // W tile: element (kk, j) is W[k0 + kk][col0 + j] (or W[col0 + j][k0 + kk] when TRANS).
    auto load_b = [&](uint32_t k0) {
        if constexpr (TRANS) {
            if constexpr (WV == 4) {
#pragma unroll
                for (int p = 0; p < B_ELEMS / 4; p++) {
                    const int idx = tid + p * kFcThreads;
                    const int j = idx / (BK / 4), k4 = (idx % (BK / 4)) * 4;
                    const uint32_t c = col0 + j, kk = k0 + k4;
                    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (c < a.n) {
                        const float* src = a.W + (uint64_t)c * a.ldw + kk;
                        if (kk + 4 <= a.k) {
                            v = *reinterpret_cast<const float4*>(src);
                        } else {
                            if (kk < a.k) v.x = src[0];
                            if (kk + 1 < a.k) v.y = src[1];
                            if (kk + 2 < a.k) v.z = src[2];
                        }
                    }
                    rb[p * 4 + 0] = v.x; rb[p * 4 + 1] = v.y; rb[p * 4 + 2] = v.z; rb[p * 4 + 3] = v.w;
                }
            } else {
#pragma unroll
                for (int p = 0; p < B_ELEMS; p++) {
                    const int idx = tid + p * kFcThreads;
                    const int j = idx / BK, kk = idx % BK;
                    const uint32_t c = col0 + j;
                    rb[p] = (c < a.n && k0 + kk < a.k) ? a.W[(uint64_t)c * a.ldw + k0 + kk] : 0.0f;
                }
            }
        } else {
#pragma unroll
            for (int p = 0; p < B_ELEMS / WV; p++) {
                const int idx = tid + p * kFcThreads;
                const int kk = idx / (BN / WV), j = (idx % (BN / WV)) * WV;
                const uint32_t c = col0 + j, kr = k0 + kk;
                float v[WV];
#pragma unroll
                for (int e = 0; e < WV; e++) v[e] = 0.0f;
                if (kr < a.k) {
                    const float* src = a.W + (uint64_t)kr * a.ldw + c;
                    if (c + WV <= a.n) {
                        if constexpr (WV == 4) {
                            const float4 t = *reinterpret_cast<const float4*>(src);
                            v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
                        } else if constexpr (WV == 2) {
                            const float2 t = *reinterpret_cast<const float2*>(src);
                            v[0] = t.x; v[1] = t.y;
                        } else {
                            v[0] = src[0];
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < WV; e++)
                            if (c + e < a.n) v[e] = src[e];
                    }
                }
#pragma unroll
                for (int e = 0; e < WV; e++) rb[p * WV + e] = v[e];
            }
        }
    };
    auto store_b = [&](int buf) {
        if constexpr (TRANS) {
            if constexpr (WV == 4) {
#pragma unroll
                for (int p = 0; p < B_ELEMS / 4; p++) {
                    const int idx = tid + p * kFcThreads;
                    const int j = idx / (BK / 4), k4 = (idx % (BK / 4)) * 4;
#pragma unroll
                    for (int c = 0; c < 4; c++) sB[buf][k4 + c][j] = rb[p * 4 + c];
                }
            } else {
#pragma unroll
                for (int p = 0; p < B_ELEMS; p++) {
                    const int idx = tid + p * kFcThreads;
                    sB[buf][idx % BK][idx / BK] = rb[p];
                }
            }
        } else {
#pragma unroll
            for (int p = 0; p < B_ELEMS / WV; p++) {
                const int idx = tid + p * kFcThreads;
                const int kk = idx / (BN / WV), j = (idx % (BN / WV)) * WV;
#pragma unroll
                for (int e = 0; e < WV; e++) sB[buf][kk][j + e] = rb[p * WV + e];
            }
        }
    };

    const uint32_t nk = (a.k + BK - 1) / BK;
    auto multiply = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            float av[MI], bv[NI];
#pragma unroll
            for (int i = 0; i < MI; i++) av[i] = sA[buf][kk + lhi][wm * 32 * MI + i * 32 + l32];
#pragma unroll
            for (int j = 0; j < NI; j++) bv[j] = sB[buf][kk + lhi][wn * 32 * NI + j * 32 + l32];
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int j = 0; j < NI; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], bv[j], acc[i][j], 0, 0, 0);
        }
    };
    // Interior tiles (the vast majority): no bounds checks, and every load is "uniform base + this lane's constant 32-bit byte
    // offset", so a k-step costs a handful of vector instructions.  That matters more than usual here: fp32 MFMA and ordinary
    // vector instructions do not overlap on this part (measured), so every VALU instruction in the loop is MFMA time lost.
    bool lean = false;
    if constexpr (!TRANS && XV == 4 && (WV == 4 || WV == 2)) {
        lean = a.fast32 && (row0 + BM <= a.batch) && (col0 + BN <= a.n) && (a.k % BK == 0);
        if (lean) {
            uint32_t offA[A_ELEMS / 4], offB[B_ELEMS / WV];
#pragma unroll
            for (int p = 0; p < A_ELEMS / 4; p++) {
                const int idx = tid + p * kFcThreads;
                offA[p] = ((row0 + idx / (BK / 4)) * a.ldx + (idx % (BK / 4)) * 4) * 4u;
            }
#pragma unroll
            for (int p = 0; p < B_ELEMS / WV; p++) {
                const int idx = tid + p * kFcThreads;
                offB[p] = ((uint32_t)(idx / (BN / WV)) * a.ldw + col0 + (idx % (BN / WV)) * WV) * 4u;
            }
            auto load_lean = [&](uint32_t k0) __attribute__((always_inline)) {
                const char* pa = reinterpret_cast<const char*>(a.X) + (uint64_t)k0 * 4;
                const char* pb = reinterpret_cast<const char*>(a.W) + (uint64_t)k0 * a.ldw * 4;
#pragma unroll
                for (int p = 0; p < A_ELEMS / 4; p++) {
                    const float4 v = *reinterpret_cast<const float4*>(pa + offA[p]);
                    ra[p * 4 + 0] = v.x; ra[p * 4 + 1] = v.y; ra[p * 4 + 2] = v.z; ra[p * 4 + 3] = v.w;
                }
#pragma unroll
                for (int p = 0; p < B_ELEMS / WV; p++) {
                    if constexpr (WV == 4) {
                        const float4 t = *reinterpret_cast<const float4*>(pb + offB[p]);
                        rb[p * 4 + 0] = t.x; rb[p * 4 + 1] = t.y; rb[p * 4 + 2] = t.z; rb[p * 4 + 3] = t.w;
                    } else {
                        const float2 t = *reinterpret_cast<const float2*>(pb + offB[p]);
                        rb[p * 2 + 0] = t.x; rb[p * 2 + 1] = t.y;
                    }
                }
            };
            load_lean(0);
            if constexpr (CAND) asm volatile("" ::"v"(bound_key));   // the bound's load is issued up here, not moved down to its use
            store_a(0);
            store_b(0);
            __syncthreads();
            auto k_step = [&](uint32_t kt, int buf) __attribute__((always_inline)) {
                if (kt + 1 < nk) load_lean((kt + 1) * BK);
                // (with two steps per trip the first step's condition is known to hold and its loads are straight-line code, which
                // the scheduler sinks to the end of the step, in front of the LDS stores that wait for them: they stay up here)
                __builtin_amdgcn_sched_barrier(0);
                multiply(buf);
                if (kt + 1 < nk) {
                    store_a(buf ^ 1);
                    store_b(buf ^ 1);
                }
                __syncthreads();
            };
            if constexpr (BK >= 16) {
                // Two k-steps per trip: each step's LDS buffer is then a constant and its addresses are immediate offsets, a
                // dozen vector instructions less per step (1.5-1.8 % at k = 512 and 1,024; with steps of 8 the longer loop body
                // costs more than that saves).
                uint32_t kt = 0;
                for (; kt + 1 < nk; kt += 2) {
                    k_step(kt, 0);
                    k_step(kt + 1, 1);
                }
                if (kt < nk) k_step(kt, 0);
            } else {
                for (uint32_t kt = 0; kt < nk; kt++) k_step(kt, (int)(kt & 1));
            }
        }
    }
    if (!lean) {
        load_a(0);
        load_b(0);
        if constexpr (CAND) asm volatile("" ::"v"(bound_key));
        store_a(0);
        store_b(0);
        __syncthreads();
        for (uint32_t kt = 0; kt < nk; kt++) {
            const int buf = kt & 1;
            if (kt + 1 < nk) {
                load_a((kt + 1) * BK);
                load_b((kt + 1) * BK);
            }
            multiply(buf);
            if (kt + 1 < nk) {
                store_a(buf ^ 1);
                store_b(buf ^ 1);
            }
            __syncthreads();
        }
    }

    __builtin_amdgcn_s_setprio(0);
    if constexpr (CAND) {
        static_assert(sizeof(sA) >= kCandLdsBytes<MI>, "the epilogue reuses the X tile's LDS");
        // (the k-loop ended with a barrier: every wavefront is done with sA)
        candidate_epilogue<MI, NI, 2, 2, CAND == 2>(acc, &sA[0][0][0], a.cand, bound_key, row0, col0, a.batch, a.n, tid, wm, wn, l32, lhi);
        return;
    }

    {
        static_assert(sizeof(sA) >= 2 * 512 * sizeof(float) && sizeof(sB) >= 2 * 512 * sizeof(float),
                      "the segment maxima are transposed through the operand tiles' LDS, two wavefronts in each");
        // (the k-loop ended with a barrier: every wavefront is done with sA / sB)
        fc_epilogue<MI, NI, ACT>(acc, a, row0 + wm * 32 * MI, col0 + wn * 32 * NI, lane,
                                 ((wave < 2) ? &sA[0][0][0] : &sB[0][0][0]) + (wave & 1) * 512);
    }
}

// Small problems (a few dozen 64 x 64 tiles, e.g. the 128-wide hidden layers at batch 1024) are bound by the chain of load
// latencies of a k-loop, not by the matrix cores.  Here a workgroup owns a 32 x 32 tile of Z and its four wavefronts split k
// four ways: every lane requests all its operands at once, straight from global memory into registers (the X row segment as
// 128-bit loads, the W column as dwords that coalesce across the 32 lanes of a half wave), one round trip instead of one
// per k-step; the four partial tiles meet in LDS.  S = k / 4 (32 or 64).
// Three bf16 planes of eight fp32 values (see fc_split_kernel below): hi = RN(x), mid = RN(x - hi), lo = RN(x - hi - mid), packed two
// to a word; infinities, NaN and what would round up to infinity stay in the first plane alone.  One 16-byte unit per plane.
__device__ __forceinline__ uint32_t bf16_rn_bits(float x)
{
    const uint32_t u = __float_as_uint(x);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

__device__ __forceinline__ void split_unit_store(const float (&x)[8], uint4* __restrict__ planes, uint64_t unit, uint64_t plane)
{
    uint32_t h[8], m[8], l[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
        if (!(fabsf(x[e]) < 3.0e38f)) {
            h[e] = __float_as_uint(x[e]) >> 16; m[e] = 0; l[e] = 0;
            if (x[e] != x[e]) h[e] |= 0x40;
            continue;
        }
        h[e] = bf16_rn_bits(x[e]);
        const float r1 = x[e] - __uint_as_float(h[e] << 16);   // exact
        m[e] = bf16_rn_bits(r1);
        const float r2 = r1 - __uint_as_float(m[e] << 16);     // exact
        l[e] = bf16_rn_bits(r2);
    }
    planes[unit] = make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
    planes[plane + unit] = make_uint4(m[0] | (m[1] << 16), m[2] | (m[3] << 16), m[4] | (m[5] << 16), m[6] | (m[7] << 16));
    planes[2 * plane + unit] = make_uint4(l[0] | (l[1] << 16), l[2] | (l[3] << 16), l[4] | (l[5] << 16), l[6] | (l[7] << 16));
}

template <int S, int ACT>
__global__ __launch_bounds__(kFcThreads) void fc_small_kernel(FcArgs a)
{
    __builtin_amdgcn_s_setprio(3);   // short kernels issue ahead of a GEMM's wavefronts that share their SIMD
    constexpr int T = S / 2;   // MFMA steps per wavefront; lane half h supplies k = base + h * T + t at step t
    __shared__ float sPart[4][16][kWave];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lhi = lane >> 5;
    const uint32_t col0 = blockIdx.x * 32, row0 = blockIdx.y * 32;
    const uint32_t kbase = wave * S + lhi * T;
    const uint32_t row = min(row0 + l32, a.batch - 1), col = min(col0 + l32, a.n - 1);   // out-of-range lanes repeat the edge; never stored

    float av[T], bv[T];
    const float* xsrc = a.X + (uint64_t)row * a.ldx + kbase;
#pragma unroll
    for (int t = 0; t < T; t += 4) {
        const float4 v = *reinterpret_cast<const float4*>(xsrc + t);
        av[t] = v.x; av[t + 1] = v.y; av[t + 2] = v.z; av[t + 3] = v.w;
    }
    const float* wsrc = a.W + (uint64_t)kbase * a.ldw + col;
#pragma unroll
    for (int t = 0; t < T; t++) bv[t] = wsrc[(uint64_t)t * a.ldw];
    const float bias = a.bias ? a.bias[col] : 0.0f;

    floatx16 acc;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.0f;
#pragma unroll
    for (int t = 0; t < T; t++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[t], bv[t], acc, 0, 0, 0);

    // every wavefront publishes its partial tile and finishes four of the sixteen accumulator registers
#pragma unroll
    for (int v = 0; v < 16; v++) sPart[wave][v][lane] = acc[v];
    __syncthreads();
    const bool col_ok = col0 + l32 < a.n;
    float y[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int v = wave * 4 + q;
        const float x = ((sPart[0][v][lane] + sPart[1][v][lane]) + (sPart[2][v][lane] + sPart[3][v][lane])) + bias;
        const uint32_t r = row0 + 8 * (v / 4) + 4 * lhi + (v % 4);   // v / 4 == wave, v % 4 == q
        y[q] = activate<ACT>(x, a.slope, a.alpha, a.lambda);
        if (col_ok && r < a.batch) a.Z[(uint64_t)r * a.ldz + col0 + l32] = y[q];
    }
    if (a.out_planes == nullptr) return;   // (the same for the whole workgroup)
    // The tile once more as planes: a unit is eight consecutive columns of one row.  The tile goes through LDS (the partial
    // tiles are done with after the barrier), 128 lanes then pack one unit each.
    __syncthreads();
    float (*sOut)[33] = reinterpret_cast<float (*)[33]>(&sPart[0][0][0]);
#pragma unroll
    for (int q = 0; q < 4; q++) sOut[8 * wave + 4 * lhi + q][l32] = col_ok ? y[q] : 0.0f;   // zeros beyond the last column: k padding
    __syncthreads();
    if (tid < 128) {
        const uint32_t rl = tid >> 2, kbl = tid & 3;
        const uint32_t r = row0 + rl, kb = col0 / 8 + kbl;
        if (r < a.batch && kb < a.out_kblocks) {
            float x[8];
#pragma unroll
            for (int e = 0; e < 8; e++) x[e] = sOut[rl][8 * kbl + e];
            split_unit_store(x, a.out_planes, (uint64_t)kb * a.out_rows_padded + r, (uint64_t)a.out_kblocks * a.out_rows_padded);
        }
    }
}

template <int S> static void launch_fc_small(const FcArgs& a)
{
    hipStream_t s = ctx().stream;
    const dim3 grid((a.n + 31) / 32, (a.batch + 31) / 32);
#define DSX_ACT_CASE(A) case A: hipLaunchKernelGGL((fc_small_kernel<S, A>), grid, dim3(kFcThreads), 0, s, a); break;
    switch (a.act) {
        DSX_ACT_CASE(DSX_ACT_SIGMOID)
        DSX_ACT_CASE(DSX_ACT_TANH)
        DSX_ACT_CASE(DSX_ACT_RELU)
        DSX_ACT_CASE(DSX_ACT_LRELU)
        DSX_ACT_CASE(DSX_ACT_ELU)
        DSX_ACT_CASE(DSX_ACT_SELU)
    default: hipLaunchKernelGGL((fc_small_kernel<S, DSX_ACT_LINEAR>), grid, dim3(kFcThreads), 0, s, a); break;
    }
#undef DSX_ACT_CASE
}

template <int MI, int NI, int BK, int XV, int WV, bool TRANS>
static void launch_fc_act(const FcArgs& a, uint32_t grid)
{
    hipStream_t s = ctx().stream;
#define DSX_ACT_CASE(A) \
    case A: hipLaunchKernelGGL((fc_gemm_kernel<MI, NI, BK, XV, WV, TRANS, A>), dim3(grid), dim3(kFcThreads), 0, s, a); break;
    switch (a.act) {
        DSX_ACT_CASE(DSX_ACT_SIGMOID)
        DSX_ACT_CASE(DSX_ACT_TANH)
        DSX_ACT_CASE(DSX_ACT_RELU)
        DSX_ACT_CASE(DSX_ACT_LRELU)
        DSX_ACT_CASE(DSX_ACT_ELU)
        DSX_ACT_CASE(DSX_ACT_SELU)
    default: hipLaunchKernelGGL((fc_gemm_kernel<MI, NI, BK, XV, WV, TRANS, DSX_ACT_LINEAR>), dim3(grid), dim3(kFcThreads), 0, s, a); break;
    }
#undef DSX_ACT_CASE
}

template <int MI, int NI, int BK> static void launch_fc_shape(FcArgs& a, int xv, int wv, bool trans)
{
    constexpr int BM = 64 * MI, BN = 64 * NI;
    a.tiles_m = (a.batch + BM - 1) / BM;
    a.tiles_n = (a.n + BN - 1) / BN;
    const uint32_t total = a.tiles_m * a.tiles_n;
    const uint32_t grid = ((total + kXcds - 1) / kXcds) * kXcds;
    if (trans) {
        if (xv == 4 && wv == 4) launch_fc_act<MI, NI, BK, 4, 4, true>(a, grid);
        else if (xv == 4) launch_fc_act<MI, NI, BK, 4, 1, true>(a, grid);
        else if (wv == 4) launch_fc_act<MI, NI, BK, 1, 4, true>(a, grid);
        else launch_fc_act<MI, NI, BK, 1, 1, true>(a, grid);
    } else if (xv == 4) {
        if (wv == 4) launch_fc_act<MI, NI, BK, 4, 4, false>(a, grid);
        else if (wv == 2) launch_fc_act<MI, NI, BK, 4, 2, false>(a, grid);
        else launch_fc_act<MI, NI, BK, 4, 1, false>(a, grid);
    } else {
        if (wv == 4) launch_fc_act<MI, NI, BK, 1, 4, false>(a, grid);
        else if (wv == 2) launch_fc_act<MI, NI, BK, 1, 2, false>(a, grid);
        else launch_fc_act<MI, NI, BK, 1, 1, false>(a, grid);
    }
}

int fc_run(const float* X, uint32_t ldx, const float* W, uint32_t ldw, int transposed, const float* bias, float* Z, uint32_t ldz,
           uint32_t batch, uint32_t k, uint32_t n, int accumulate, uint32_t activation, const dsx_act_params* params, float* seg_max,
           uint32_t* seg_width, void* out_planes)
{
    if (seg_width) *seg_width = 0;
    FcArgs a{};
    a.X = X; a.W = W; a.bias = bias; a.Z = Z;
    a.ldx = ldx; a.ldw = ldw; a.ldz = ldz;
    a.batch = batch; a.k = k; a.n = n;
    a.accumulate = accumulate;
    a.act = activation;
    a.slope = params ? params->slope : 0.01f;
    a.alpha = params ? params->alpha : 1.0f;
    a.lambda = params ? params->lambda : 1.0f;
    // the lean path's per-lane offsets: (row * ldx + k4) * 4 into X, (kk * ldw + column) * 4 with kk < 32 into a k-slice of W
    a.fast32 = ((uint64_t)(batch + 128) * ldx * 4 < (1ull << 32)) && ((32ull * ldw + n + 128) * 4 < (1ull << 32));
    const int xv = (((uintptr_t)X % 16) == 0 && (ldx % 4) == 0) ? 4 : 1;
    int wv = 1;
    if (((uintptr_t)W % 16) == 0 && (ldw % 4) == 0) wv = 4;
    else if (!transposed && ((uintptr_t)W % 8) == 0 && (ldw % 2) == 0) wv = 2;
    // Large tiles when they still give every CU a few workgroups, small tiles otherwise.
    const uint64_t big_tiles = (uint64_t)((batch + 127) / 128) * ((n + 127) / 128);
    if (big_tiles >= (uint64_t)ctx().num_cus * 2) {
        if (seg_max && seg_width && !accumulate) {   // maxima of sums still to be accumulated into would be of no use
            a.seg_max = seg_max;
            a.nseg = (n + 63) / 64;
            *seg_width = 64;
        }
        // Short sums (the wide layer behind a narrow one) are staged eight k-steps at a time: the multiplications cost the same,
        // and the kernels of other streams that share the CUs find 17 KiB of LDS taken per workgroup instead of 34.
        if (k <= 256) launch_fc_shape<2, 2, 8>(a, xv, wv, transposed != 0);
        else launch_fc_shape<2, 2, 16>(a, xv, wv, transposed != 0);
    } else if (!transposed && !accumulate && xv == 4 && (k == 128 || k == 256) && (uint64_t)batch * n <= (1u << 20)) {
        if (out_planes) {   // the result also as the next layer's planes, written by the same workgroups
            a.out_planes = reinterpret_cast<uint4*>(out_planes);
            a.out_rows_padded = split_rows_padded(batch);
            a.out_kblocks = (n + 15) / 16 * 2;
            out_planes = nullptr;
        }
        if (k == 128) launch_fc_small<32>(a);   // latency bound: all operands in one round trip
        else launch_fc_small<64>(a);
    } else
        launch_fc_shape<1, 1, 32>(a, xv, wv, transposed != 0);   // few workgroups: deep k-steps, fewer barrier round trips
    DSX_LAUNCH_CHECK("fc_gemm_kernel");
    if (out_planes) return fc_split_planes_run(Z, ldz, 1, batch, n, out_planes);   // every other kernel: a launch of its own
    return DSX_OK;
}

// Scores of queries[batch][k] against n columns of W, compared with the rows' bounds instead of stored (FcArgs, candidate
// mode).  The caller guarantees 16-byte aligned operands with pitches that are multiples of four floats.
int fc_candidates_run(const float* X, uint32_t ldx, const float* W, uint32_t ldw, uint32_t batch, uint32_t k, uint32_t n,
                      const CandArgs& cand)
{
    FcArgs a{};
    a.X = X; a.W = W;
    a.ldx = ldx; a.ldw = ldw;
    a.batch = batch; a.k = k; a.n = n;
    a.act = DSX_ACT_LINEAR;
    a.fast32 = ((uint64_t)(batch + 128) * ldx * 4 < (1ull << 32)) && ((32ull * ldw + n + 128) * 4 < (1ull << 32));
    a.cand = cand;
    a.tiles_m = (batch + 127) / 128;
    a.tiles_n = (n + 127) / 128;
    const uint32_t total = a.tiles_m * a.tiles_n;
    const uint32_t grid = ((total + kXcds - 1) / kXcds) * kXcds;
    hipLaunchKernelGGL((fc_gemm_kernel<2, 2, 16, 4, 4, false, DSX_ACT_LINEAR, 1>), dim3(grid), dim3(kFcThreads), 0, ctx().stream, a);
    DSX_LAUNCH_CHECK("fc_gemm_kernel (candidates)");
    return DSX_OK;
}

// The same for a layer: Z = act(bias + X.W) is not stored; cand.act / slope / alpha / lambda describe the activation and
// cand.row_bound holds keys of activated scores.  X must be 16-byte aligned with a pitch that is a multiple of four floats; W may
// be aligned to 16, 8 or 4 bytes (a 27,278-wide row-major matrix is 8-byte aligned).
int fc_layer_candidates_run(const float* X, uint32_t ldx, const float* W, uint32_t ldw, const float* bias, uint32_t batch, uint32_t k,
                            uint32_t n, const CandArgs& cand)
{
    FcArgs a{};
    a.X = X; a.W = W; a.bias = bias;
    a.ldx = ldx; a.ldw = ldw;
    a.batch = batch; a.k = k; a.n = n;
    a.act = DSX_ACT_LINEAR;
    a.fast32 = ((uint64_t)(batch + 128) * ldx * 4 < (1ull << 32)) && ((32ull * ldw + n + 128) * 4 < (1ull << 32));
    a.cand = cand;
    a.tiles_m = (batch + 127) / 128;
    a.tiles_n = (n + 127) / 128;
    const uint32_t total = a.tiles_m * a.tiles_n;
    const dim3 grid(((total + kXcds - 1) / kXcds) * kXcds);
    hipStream_t s = ctx().stream;
    if (((uintptr_t)W % 16) == 0 && (ldw % 4) == 0)
        hipLaunchKernelGGL((fc_gemm_kernel<2, 2, 16, 4, 4, false, DSX_ACT_LINEAR, 2>), grid, dim3(kFcThreads), 0, s, a);
    else if (((uintptr_t)W % 8) == 0 && (ldw % 2) == 0)
        hipLaunchKernelGGL((fc_gemm_kernel<2, 2, 16, 4, 2, false, DSX_ACT_LINEAR, 2>), grid, dim3(kFcThreads), 0, s, a);
    else
        hipLaunchKernelGGL((fc_gemm_kernel<2, 2, 16, 4, 1, false, DSX_ACT_LINEAR, 2>), grid, dim3(kFcThreads), 0, s, a);
    DSX_LAUNCH_CHECK("fc_gemm_kernel (layer candidates)");
    return DSX_OK;
}

// ---------------------------------------------------------------------------------------------------------------------
// fp32 products from bf16 matrix instructions (a mode the caller asks for; the kernels above multiply in fp32).
// An fp32 value is the exact sum of three bf16 values, hi + mid + lo (3 x 8 significant bits, each rounded to nearest from what
// the ones before left).  Of the nine products of two such sums, the six that reach 2^-24 of the full product are accumulated
// in fp32 by v_mfma_f32_32x32x16_bf16, smallest first: twelve matrix-core cycles per k and 32 x 32 block where
// v_mfma_f32_32x32x2_f32 takes thirty-two.  What is dropped (mid.lo, lo.mid, lo.lo) is below 2^-25 of a product, less than the
// rounding of the product itself in fp32; measured against fp64, the sums are as close as the fp32 kernel's.
// Operands come pre-split ("planes"): plane p, block kb of eight consecutive k, row r (a row of X or a column of W) is one
// 16-byte unit at ((p * kblocks + kb) * rows_padded + r), rows padded to 128 and k to 16 with zeros, so that a lane's MFMA
// operand is one 128-bit read, the 128 rows of a tile are 2 KiB of consecutive memory and no load needs a bounds check.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));   // (a native vector: arrays of it stay in registers)

// src element (r, kk) is src[r * stride_r + kk * stride_k].  One lane per (block of eight k, row); consecutive lanes take
// consecutive rows (a [k][n] weight matrix is read along n, the planes are written 16 bytes per lane, consecutively).
__global__ __launch_bounds__(256) void fc_split_kernel(const float* __restrict__ src, uint64_t stride_r, uint64_t stride_k, uint32_t rows,
                                                        uint32_t k, uint32_t rows_padded, uint32_t kblocks, uint4* __restrict__ planes)
{
    const uint64_t id = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= (uint64_t)rows_padded * kblocks) return;
    const uint32_t r = (uint32_t)(id % rows_padded), kb = (uint32_t)(id / rows_padded);
    float x[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const uint32_t kk = kb * 8 + e;
        x[e] = (r < rows && kk < k) ? src[r * stride_r + kk * stride_k] : 0.0f;
    }
    split_unit_store(x, planes, (uint64_t)kb * rows_padded + r, (uint64_t)kblocks * rows_padded);
}

struct FcSplitArgs {
    const u32x4* Xs;
    const u32x4* Ws;
    uint32_t xrows, wrows, kblocks;   // padded rows of the two sets of planes; blocks of eight k (an even number)
    uint32_t wcol0;                   // the product's first column is row wcol0 of the W planes (a multiple of 128)
};

// Z = act(acc? + bias + X . W) as fc_gemm_kernel<2, 2, ...> computes it (same tile order, same epilogue), from planes.
// A k-step is one MFMA depth (16), its operand units double buffered in LDS.  MH = 1: a 128 x 128 tile, 2 x 2 wavefronts of
// 64 x 64, 24 KiB of units per step, three workgroups per CU.  MH = 2: a 256 x 128 tile, wavefronts of 128 x 64 (eight
// accumulators: 0.375 fragment reads per MFMA instead of 0.5, and three quarters of the operand traffic per product), 36 KiB
// per step, two workgroups per CU.
// CAND (MH = 1 only): the candidate modes of fc_gemm_kernel, the scores compared with the rows' bounds instead of stored:
// 1 = exact KNN, 2 = a layer (the sums start from the bias, pre-activation sums against bounds derived from activated scores).
template <int ACT, int MH, int CAND = 0>
__global__ __launch_bounds__(kFcThreads, MH == 1 ? 3 : 2) void fc_gemm_split_kernel(FcArgs a, FcSplitArgs sp)
{
    static_assert(CAND == 0 || MH == 1, "the candidate epilogue works on tiles of 128 rows");
    constexpr int BM = 128 * MH;
    __shared__ u32x4 sA[2][3][2][BM];
    __shared__ u32x4 sB[2][3][2][128];
    const uint32_t total = a.tiles_m * a.tiles_n;
    uint32_t wg = blockIdx.x;
    {
        const uint32_t per_xcd = (total + kXcds - 1) / kXcds;
        const uint32_t xcd = wg % kXcds, local = wg / kXcds;
        wg = xcd * per_xcd + local;
        if (local >= per_xcd || wg >= total) return;
    }
    const uint32_t tm = wg % a.tiles_m, tn = a.tiles_n - 1 - wg / a.tiles_m;
    const uint32_t row0 = tm * BM, col0 = tn * 128;
    __builtin_amdgcn_s_setprio(1);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lhi = lane >> 5;

    floatx16 acc[MH][2][2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        float start = 0.0f;
        if constexpr (CAND == 2) {   // every register of a lane belongs to column l32 of its block: the sums start from the bias
            const uint32_t c = col0 + wn * 64 + j * 32 + l32;
            if (a.bias && c < a.n) start = a.bias[c];
        }
#pragma unroll
        for (int h = 0; h < MH; h++)
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[h][i][j][v] = start;
    }
    uint32_t bound_key = 0;
    if constexpr (CAND) bound_key = candidate_bound_prefetch<2>(a.cand, row0, a.batch, tid);

    // Every load is "plane base (uniform) + this lane's 32-bit byte offset", the offset advancing by a uniform step per k-step
    // (a plane is smaller than 4 GiB, the host checks): two vector additions per step instead of 64-bit address arithmetic.
    // W: lane (half, row) moves one unit per plane.  X: the same for MH = 1; for MH = 2 a lane moves both halves of its row.
    const int srow = tid & 127, shalf = tid >> 7;
    const uint64_t xplane = (uint64_t)sp.kblocks * sp.xrows * 16, wplane = (uint64_t)sp.kblocks * sp.wrows * 16;
    const char* xbase[3];
    const char* wbase[3];
#pragma unroll
    for (int p = 0; p < 3; p++) {
        xbase[p] = reinterpret_cast<const char*>(sp.Xs) + p * xplane;
        wbase[p] = reinterpret_cast<const char*>(sp.Ws) + p * wplane;
    }
    uint32_t xoff = (MH == 1) ? (shalf * sp.xrows + row0 + srow) * 16u : (row0 + tid) * 16u;
    uint32_t woff = (shalf * sp.wrows + sp.wcol0 + col0 + srow) * 16u;
    const uint32_t xhalf = sp.xrows * 16u;
    const uint32_t xstep = 2u * sp.xrows * 16u, wstep = 2u * sp.wrows * 16u;
    u32x4 ra[3 * MH], rb[3];
    auto load = [&]() __attribute__((always_inline)) {   // the next k-step's units
#pragma unroll
        for (int p = 0; p < 3; p++) {
            if constexpr (MH == 1) {
                ra[p] = *reinterpret_cast<const u32x4*>(xbase[p] + xoff);
            } else {
                ra[2 * p] = *reinterpret_cast<const u32x4*>(xbase[p] + xoff);
                ra[2 * p + 1] = *reinterpret_cast<const u32x4*>(xbase[p] + xoff + xhalf);
            }
            rb[p] = *reinterpret_cast<const u32x4*>(wbase[p] + woff);
        }
        xoff += xstep;
        woff += wstep;
    };
    auto store = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < 3; p++) {
            if constexpr (MH == 1) {
                sA[buf][p][shalf][srow] = ra[p];
            } else {
                sA[buf][p][0][tid] = ra[2 * p];
                sA[buf][p][1][tid] = ra[2 * p + 1];
            }
            sB[buf][p][shalf][srow] = rb[p];
        }
    };
    auto multiply = [&](int buf) __attribute__((always_inline)) {
        bf16x8 fb[2][3];
#pragma unroll
        for (int p = 0; p < 3; p++)
#pragma unroll
            for (int j = 0; j < 2; j++) fb[j][p] = __builtin_bit_cast(bf16x8, sB[buf][p][lhi][wn * 64 + j * 32 + l32]);
#pragma unroll
        for (int h = 0; h < MH; h++) {
            bf16x8 fa[2][3];
#pragma unroll
            for (int p = 0; p < 3; p++)
#pragma unroll
                for (int i = 0; i < 2; i++) fa[i][p] = __builtin_bit_cast(bf16x8, sA[buf][p][lhi][wm * 64 * MH + h * 64 + i * 32 + l32]);
            // (plane of X, plane of W): lo.hi, hi.lo, mid.mid, mid.hi, hi.mid, hi.hi; the four accumulators take turns
#define DSX_TERM(PX, PW)                                                                                                   \
    _Pragma("unroll") for (int i = 0; i < 2; i++) _Pragma("unroll") for (int j = 0; j < 2; j++)                            \
        acc[h][i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i][PX], fb[j][PW], acc[h][i][j], 0, 0, 0);
            DSX_TERM(2, 0) DSX_TERM(0, 2) DSX_TERM(1, 1) DSX_TERM(1, 0) DSX_TERM(0, 1) DSX_TERM(0, 0)
#undef DSX_TERM
        }
    };
    const uint32_t nk = sp.kblocks / 2;
    load();
    if constexpr (CAND) asm volatile("" ::"v"(bound_key));   // the bound's load is issued up here, not moved down to its use
    store(0);
    __syncthreads();
    for (uint32_t kt = 0; kt < nk; kt++) {
        const int buf = kt & 1;
        // (unconditional, so that the staging registers stay registers: the last step loads its own units again, and they go
        // where nobody reads them)
        if (kt + 1 == nk) {
            xoff -= xstep;
            woff -= wstep;
        }
        load();
        // (the loads stay up here: left to itself the scheduler sinks them to the end of the step, right in front of the LDS
        // stores that wait for them, and every step then pays a round trip to L2)
        __builtin_amdgcn_sched_barrier(0);
        multiply(buf);
        store(buf ^ 1);
        __syncthreads();
    }
    __builtin_amdgcn_s_setprio(0);
    if constexpr (CAND) {
        static_assert(sizeof(sA) >= kCandLdsBytes<2>, "the epilogue reuses the X tile's LDS");
        // (the k-loop ended with a barrier: every wavefront is done with sA)
        candidate_epilogue<2, 2, 2, 2, CAND == 2>(acc[0], reinterpret_cast<float*>(&sA[0][0][0][0]), a.cand, bound_key, row0, col0, a.batch, a.n,
                                                  tid, wm, wn, l32, lhi);
        return;
    }
    static_assert(sizeof(sA) >= 2 * 512 * sizeof(float) && sizeof(sB) >= 2 * 512 * sizeof(float),
                  "the segment maxima are transposed through the operand tiles' LDS, two wavefronts in each");
    float* sT = reinterpret_cast<float*>((wave < 2) ? &sA[0][0][0][0] : &sB[0][0][0][0]) + (wave & 1) * 512;
#pragma unroll
    for (int h = 0; h < MH; h++) fc_epilogue<2, 2, ACT>(acc[h], a, row0 + wm * 64 * MH + h * 64, col0 + wn * 64, lane, sT);
}

uint32_t split_rows_padded(uint32_t rows) { return (rows + 255) / 256 * 256; }
static inline uint32_t split_kblocks(uint32_t k) { return (k + 15) / 16 * 2; }
uint64_t split_plane_bytes(uint32_t rows, uint32_t k) { return 3ull * split_rows_padded(rows) * split_kblocks(k) * 16; }

int fc_split_planes_run(const float* src, uint64_t stride_r, uint64_t stride_k, uint32_t rows, uint32_t k, void* planes)
{
    const uint32_t rp = split_rows_padded(rows), kb = split_kblocks(k);
    const uint64_t units = (uint64_t)rp * kb;
    hipLaunchKernelGGL(fc_split_kernel, dim3((uint32_t)((units + 255) / 256)), dim3(256), 0, ctx().stream, src, stride_r, stride_k, rows, k, rp,
                       kb, reinterpret_cast<uint4*>(planes));
    DSX_LAUNCH_CHECK("fc_split_kernel");
    return DSX_OK;
}

static int split_planes_fit(uint32_t xrows, uint32_t wrows, uint32_t kblocks, uint32_t wcol0, uint32_t n)
{
    if ((uint64_t)kblocks * xrows * 16 >= (1ull << 32) || (uint64_t)kblocks * wrows * 16 >= (1ull << 32))
        return set_error(DSX_EINVAL, "dsx_fc_forward_split: a plane of 4 GiB or more (rows padded to 256 x k padded to 16 x 2 bytes)");
    if (wcol0 % 128 != 0 || (uint64_t)wcol0 + (n + 127) / 128 * 128 > wrows)
        return set_error(DSX_EINVAL, "dsx_fc_forward_split: columns %u .. %u + %u of planes of %u rows", wcol0, wcol0, n, wrows);
    return DSX_OK;
}

// Ws: planes of wrows (padded) rows; the product's n columns are rows wcol0 .. wcol0 + n of them.
int fc_split_run(const void* Xs, const void* Ws, uint32_t wrows, uint32_t wcol0, const float* bias, float* Z, uint32_t ldz, uint32_t batch,
                 uint32_t k, uint32_t n, int accumulate, uint32_t activation, const dsx_act_params* params, float* seg_max,
                 uint32_t* seg_width)
{
    if (seg_width) *seg_width = 0;
    FcArgs a{};
    a.bias = bias; a.Z = Z; a.ldz = ldz;
    a.batch = batch; a.k = k; a.n = n;
    a.accumulate = accumulate;
    a.act = activation;
    a.slope = params ? params->slope : 0.01f;
    a.alpha = params ? params->alpha : 1.0f;
    a.lambda = params ? params->lambda : 1.0f;
    a.tiles_n = (n + 127) / 128;
    // 256-row tiles for long sums, when they still give every CU its two workgroups twice over (4,096 x 512 x 262,144: 5,410
    // against 5,730 us; with k = 128 the epilogue dominates and the smaller tiles' third workgroup per CU is worth more)
    int mh = (k >= 512 && (uint64_t)((batch + 255) / 256) * a.tiles_n >= 4ull * ctx().num_cus) ? 2 : 1;
    if (ctx().knobs.split_tile_rows) mh = ctx().knobs.split_tile_rows == 256 ? 2 : 1;
    a.tiles_m = (batch + 128 * mh - 1) / (128 * mh);
    if (seg_max && seg_width && !accumulate) {
        a.seg_max = seg_max;
        a.nseg = (n + 63) / 64;
        *seg_width = 64;
    }
    FcSplitArgs sp{reinterpret_cast<const u32x4*>(Xs), reinterpret_cast<const u32x4*>(Ws), split_rows_padded(batch), wrows, split_kblocks(k), wcol0};
    if (int rc = split_planes_fit(sp.xrows, sp.wrows, sp.kblocks, wcol0, n)) return rc;
    const uint32_t total = a.tiles_m * a.tiles_n;
    const dim3 grid(((total + kXcds - 1) / kXcds) * kXcds);
    hipStream_t s = ctx().stream;
#define DSX_ACT_CASE(A)                                                                                      \
    case A:                                                                                                  \
        if (mh == 2) hipLaunchKernelGGL((fc_gemm_split_kernel<A, 2>), grid, dim3(kFcThreads), 0, s, a, sp); \
        else hipLaunchKernelGGL((fc_gemm_split_kernel<A, 1>), grid, dim3(kFcThreads), 0, s, a, sp);         \
        break;
    switch (a.act) {
        DSX_ACT_CASE(DSX_ACT_SIGMOID)
        DSX_ACT_CASE(DSX_ACT_TANH)
        DSX_ACT_CASE(DSX_ACT_RELU)
        DSX_ACT_CASE(DSX_ACT_LRELU)
        DSX_ACT_CASE(DSX_ACT_ELU)
        DSX_ACT_CASE(DSX_ACT_SELU)
    default:
        if (mh == 2) hipLaunchKernelGGL((fc_gemm_split_kernel<DSX_ACT_LINEAR, 2>), grid, dim3(kFcThreads), 0, s, a, sp);
        else hipLaunchKernelGGL((fc_gemm_split_kernel<DSX_ACT_LINEAR, 1>), grid, dim3(kFcThreads), 0, s, a, sp);
        break;
    }
#undef DSX_ACT_CASE
    DSX_LAUNCH_CHECK("fc_gemm_split_kernel");
    return DSX_OK;
}

// Candidate modes: scores of X's planes against columns wcol0 .. wcol0 + n of the W planes, compared with the rows' bounds
// (CandArgs) instead of stored.  layer: Z = act(bias + X.W) as fc_layer_candidates_run (cand.act etc. describe the activation,
// bias points at the window's first column); otherwise plain inner products (exact KNN).
int fc_split_candidates_run(const void* Xs, const void* Ws, uint32_t wrows, uint32_t wcol0, uint32_t batch, uint32_t k, uint32_t n,
                            const CandArgs& cand, bool layer, const float* bias)
{
    FcArgs a{};
    a.bias = bias;   // layer mode: of the window's first column
    a.batch = batch; a.k = k; a.n = n;
    a.act = DSX_ACT_LINEAR;
    a.cand = cand;
    a.tiles_m = (batch + 127) / 128;
    a.tiles_n = (n + 127) / 128;
    FcSplitArgs sp{reinterpret_cast<const u32x4*>(Xs), reinterpret_cast<const u32x4*>(Ws), split_rows_padded(batch), wrows, split_kblocks(k), wcol0};
    if (int rc = split_planes_fit(sp.xrows, sp.wrows, sp.kblocks, wcol0, n)) return rc;
    const uint32_t total = a.tiles_m * a.tiles_n;
    const dim3 grid(((total + kXcds - 1) / kXcds) * kXcds);
    if (layer) hipLaunchKernelGGL((fc_gemm_split_kernel<DSX_ACT_LINEAR, 1, 2>), grid, dim3(kFcThreads), 0, ctx().stream, a, sp);
    else hipLaunchKernelGGL((fc_gemm_split_kernel<DSX_ACT_LINEAR, 1, 1>), grid, dim3(kFcThreads), 0, ctx().stream, a, sp);
    DSX_LAUNCH_CHECK("fc_gemm_split_kernel (candidates)");
    return DSX_OK;
}

// ---------------------------------------------------------------------------------------------------------------------
// Stand-alone activations (used when a layer has several sources, so the GEMM epilogue cannot apply them).

__global__ __launch_bounds__(256) void activation_kernel(float* z, uint64_t size, uint32_t act, float slope, float alpha, float lambda)
{
    uint64_t pos = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t step = (uint64_t)gridDim.x * blockDim.x;
    for (; pos < size; pos += step) z[pos] = activate_rt(z[pos], act, slope, alpha, lambda);
}

// Row softmax (engine/kActivation.cu:155-236): a = min(1, exp(x - max) / sum exp(x - max)); one workgroup per row.
__global__ __launch_bounds__(256) void softmax_kernel(float* z, uint32_t stride)
{
    __shared__ float sRed[256 / kWave];
    float* row = z + (uint64_t)blockIdx.x * stride;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float m = -__builtin_inff();
    for (uint32_t j = threadIdx.x; j < stride; j += 256) m = fmaxf(m, row[j]);
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, kWave));
    if (lane == 0) sRed[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(sRed[0], sRed[1]), fmaxf(sRed[2], sRed[3]));
    __syncthreads();
    float s = 0.0f;
    for (uint32_t j = threadIdx.x; j < stride; j += 256) s += __expf(row[j] - m);
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, kWave);
    if (lane == 0) sRed[wave] = s;
    __syncthreads();
    s = (sRed[0] + sRed[1]) + (sRed[2] + sRed[3]);
    const float inv = 1.0f / s;
    for (uint32_t j = threadIdx.x; j < stride; j += 256) row[j] = fminf(1.0f, __expf(row[j] - m) * inv);
}

}  // namespace dsx

using namespace dsx;

extern "C" {

int dsx_fc_forward(const float* X, uint32_t ldx, const float* W, int transposed, const float* bias, float* Z, uint32_t ldz,
                   uint32_t batch, uint32_t k, uint32_t n, int accumulate, uint32_t activation, const dsx_act_params* params)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(X && W && Z, "dsx_fc_forward: null device pointer");
    DSX_CHECK_ARG(k > 0 && n > 0, "dsx_fc_forward: k = %u, n = %u", k, n);
    DSX_CHECK_ARG(ldx >= k && ldz >= n, "dsx_fc_forward: row pitch smaller than the row (ldx %u < k %u or ldz %u < n %u)", ldx, k, ldz, n);
    DSX_CHECK_ARG(is_elementwise_activation(activation), "dsx_fc_forward: activation %u is a row operation; pass DSX_ACT_LINEAR and call dsx_activation", activation);
    if (batch == 0) return DSX_OK;
    return fc_run(X, ldx, W, transposed ? k : n, transposed, bias, Z, ldz, batch, k, n, accumulate, activation, params);
}

int dsx_fc_forward_planes(const float* X, uint32_t ldx, const float* W, int transposed, const float* bias, float* Z, uint32_t ldz,
                          uint32_t batch, uint32_t k, uint32_t n, uint32_t activation, const dsx_act_params* params, void* z_planes)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(X && W && Z && z_planes, "dsx_fc_forward_planes: null device pointer");
    DSX_CHECK_ARG(((uintptr_t)z_planes % 16) == 0, "dsx_fc_forward_planes: planes must be 16-byte aligned");
    DSX_CHECK_ARG(k > 0 && n > 0, "dsx_fc_forward_planes: k = %u, n = %u", k, n);
    DSX_CHECK_ARG(ldx >= k && ldz >= n, "dsx_fc_forward_planes: row pitch smaller than the row (ldx %u < k %u or ldz %u < n %u)", ldx, k, ldz, n);
    DSX_CHECK_ARG(is_elementwise_activation(activation), "dsx_fc_forward_planes: activation %u is a row operation", activation);
    if (batch == 0) return DSX_OK;
    return fc_run(X, ldx, W, transposed ? k : n, transposed, bias, Z, ldz, batch, k, n, 0, activation, params, nullptr, nullptr, z_planes);
}

int dsx_fc_forward_segmax(const float* X, uint32_t ldx, const float* W, int transposed, const float* bias, float* Z, uint32_t ldz,
                          uint32_t batch, uint32_t k, uint32_t n, uint32_t activation, const dsx_act_params* params, float* seg_max,
                          uint32_t* seg_width)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(X && W && Z && seg_max && seg_width, "dsx_fc_forward_segmax: null pointer");
    DSX_CHECK_ARG(k > 0 && n > 0, "dsx_fc_forward_segmax: k = %u, n = %u", k, n);
    DSX_CHECK_ARG(ldx >= k && ldz >= n, "dsx_fc_forward_segmax: row pitch smaller than the row (ldx %u < k %u or ldz %u < n %u)", ldx, k, ldz, n);
    DSX_CHECK_ARG(is_elementwise_activation(activation), "dsx_fc_forward_segmax: activation %u is a row operation", activation);
    *seg_width = 0;
    if (batch == 0) return DSX_OK;
    return fc_run(X, ldx, W, transposed ? k : n, transposed, bias, Z, ldz, batch, k, n, 0, activation, params, seg_max, seg_width);
}

uint64_t dsx_fc_split_bytes(uint32_t rows, uint32_t k)
{
    return split_plane_bytes(rows, k);
}

int dsx_fc_split(const float* src, uint32_t ld, int k_major, uint32_t rows, uint32_t k, void* planes)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(src && planes, "dsx_fc_split: null device pointer");
    DSX_CHECK_ARG(((uintptr_t)planes % 16) == 0, "dsx_fc_split: planes must be 16-byte aligned");
    DSX_CHECK_ARG(rows > 0 && k > 0 && ld >= (k_major ? rows : k), "dsx_fc_split: rows = %u, k = %u, ld = %u", rows, k, ld);
    return k_major ? fc_split_planes_run(src, 1, ld, rows, k, planes) : fc_split_planes_run(src, ld, 1, rows, k, planes);
}

int dsx_testing_set_split_tile_rows(uint32_t rows)
{
    if (rows != 0 && rows != 128 && rows != 256) return set_error(DSX_EINVAL, "dsx_testing_set_split_tile_rows: %u (0, 128 or 256)", rows);
    ctx().knobs.split_tile_rows = rows;
    return DSX_OK;
}

int dsx_fc_forward_split(const void* x_planes, const void* w_planes, const float* bias, float* Z, uint32_t ldz, uint32_t batch, uint32_t k,
                         uint32_t n, int accumulate, uint32_t activation, const dsx_act_params* params, float* seg_max, uint32_t* seg_width)
{
    DSX_REQUIRE_INIT();
    if (seg_width) *seg_width = 0;
    DSX_CHECK_ARG(x_planes && w_planes && Z, "dsx_fc_forward_split: null device pointer");
    DSX_CHECK_ARG(((uintptr_t)x_planes % 16) == 0 && ((uintptr_t)w_planes % 16) == 0, "dsx_fc_forward_split: planes must be 16-byte aligned");
    DSX_CHECK_ARG(k > 0 && n > 0 && ldz >= n, "dsx_fc_forward_split: k = %u, n = %u, ldz = %u", k, n, ldz);
    DSX_CHECK_ARG(is_elementwise_activation(activation), "dsx_fc_forward_split: activation %u is a row operation; pass DSX_ACT_LINEAR and call dsx_activation", activation);
    DSX_CHECK_ARG((seg_max == NULL) == (seg_width == NULL), "dsx_fc_forward_split: seg_max and seg_width go together");
    if (batch == 0) return DSX_OK;
    return fc_split_run(x_planes, w_planes, split_rows_padded(n), 0, bias, Z, ldz, batch, k, n, accumulate, activation, params, seg_max, seg_width);
}

int dsx_activation(float* unit, uint32_t batch, uint32_t stride, uint32_t activation, const dsx_act_params* params)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(unit && stride > 0, "dsx_activation: null unit or zero stride");
    if (batch == 0) return DSX_OK;
    if (activation == DSX_ACT_SOFTMAX) {
        hipLaunchKernelGGL(softmax_kernel, dim3(batch), dim3(256), 0, ctx().stream, unit, stride);
        DSX_LAUNCH_CHECK("softmax_kernel");
        return DSX_OK;
    }
    switch (activation) {
    case DSX_ACT_SIGMOID:
    case DSX_ACT_TANH:
    case DSX_ACT_RELU:
    case DSX_ACT_LRELU:
    case DSX_ACT_ELU:
    case DSX_ACT_SELU: break;
    default: return DSX_OK;   // CalculateActivation (engine/NNLayer.cpp:1646-1683) does nothing for the other kinds
    }
    const uint64_t size = (uint64_t)batch * stride;
    uint64_t blocks = (size + 1023) / 1024;
    const uint64_t cap = (uint64_t)ctx().num_cus * 32;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(activation_kernel, dim3((uint32_t)blocks), dim3(256), 0, ctx().stream, unit, size, activation,
                       params ? params->slope : 0.01f, params ? params->alpha : 1.0f, params ? params->lambda : 1.0f);
    DSX_LAUNCH_CHECK("activation_kernel");
    return DSX_OK;
}

}  // extern "C"
