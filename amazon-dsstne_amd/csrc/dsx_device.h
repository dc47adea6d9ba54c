// dsx_device.h — device-side helpers shared by the kernels of libdsx_hip.so (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>
#include "dsx.h"

namespace dsx {

constexpr int kWave = 64;

// Activation functions of engine/kActivation.cu:46-153, applied in the epilogue of the producing kernel.
template <int ACT>
__device__ __forceinline__ float activate(float x, float slope, float alpha, float lambda)
{
    if constexpr (ACT == DSX_ACT_SIGMOID) {
        // v_exp_f32 + v_rcp_f32 (about 1 ulp each): the IEEE division sequence would triple the epilogue's instruction count
        return __builtin_amdgcn_rcpf(1.0f + __expf(-x));
    } else if constexpr (ACT == DSX_ACT_TANH) {
        return tanhf(x);
    } else if constexpr (ACT == DSX_ACT_RELU) {
        return fmaxf(0.0f, x);
    } else if constexpr (ACT == DSX_ACT_LRELU) {
        return fmaxf(x, x * slope);
    } else if constexpr (ACT == DSX_ACT_ELU) {
        return (x > 0.0f) ? x : alpha * (expf(x) - 1.0f);   // full-precision exp: exp(x) - 1 cancels near 0
    } else if constexpr (ACT == DSX_ACT_SELU) {
        return (x > 0.0f) ? lambda * x : lambda * alpha * (expf(x) - 1.0f);
    } else {
        return x;
    }
}

__device__ __forceinline__ float activate_rt(float x, uint32_t act, float slope, float alpha, float lambda)
{
    switch (act) {
    case DSX_ACT_SIGMOID: return activate<DSX_ACT_SIGMOID>(x, slope, alpha, lambda);
    case DSX_ACT_TANH: return activate<DSX_ACT_TANH>(x, slope, alpha, lambda);
    case DSX_ACT_RELU: return activate<DSX_ACT_RELU>(x, slope, alpha, lambda);
    case DSX_ACT_LRELU: return activate<DSX_ACT_LRELU>(x, slope, alpha, lambda);
    case DSX_ACT_ELU: return activate<DSX_ACT_ELU>(x, slope, alpha, lambda);
    case DSX_ACT_SELU: return activate<DSX_ACT_SELU>(x, slope, alpha, lambda);
    default: return x;
    }
}

// Unsigned key with the order of the scores (NaN patterns land above +inf or below -inf; callers keep NaN out).
__device__ __forceinline__ uint32_t score_key(float key)
{
    key += 0.0f;   // -0.0 -> +0.0 so that both zeros tie and fall back to the column order
    uint32_t u = __float_as_uint(key);
    u ^= (uint32_t)((int32_t)u >> 31) | 0x80000000u;
    return u;
}

__device__ __forceinline__ float key_score(uint32_t u)
{
    u ^= ((u >> 31) - 1u) | 0x80000000u;
    return __uint_as_float(u);
}

typedef float floatx16 __attribute__((ext_vector_type(16)));

// Candidate mode of the score kernels (exact nearest-neighbour search).  A score whose key reaches row_bound[row] is appended
// as a packed word (key << 32 | ~(col_offset + column)) to the row's list cand[row][cand_cap]; cand_count[row] counts the
// appends, and *overflow is set when a list is full.
struct CandArgs {
    const uint32_t* row_bound;
    uint64_t* cand;
    uint32_t* cand_count;
    uint32_t cand_cap;
    uint32_t col_offset;
    uint32_t* overflow;
    // Layer mode (template flag PRE of candidate_epilogue): the accumulators hold pre-activation sums z (bias included), the
    // bounds are keys of activated scores; see preactivation_bound.
    uint32_t act;
    float slope, alpha, lambda;
};

// Layer mode of the candidate epilogue.  The k-th best score B of a row is known as an activated value, the tile holds
// pre-activation sums z.  For a non-decreasing activation every z with act(z) >= B lies above any point zb with
// act(zb) < B, so "z >= zb" admits a superset of what "act(z) >= B" admits, and only the few survivors are activated.  zb is
// found by inverting the activation a little below B and stepping down until the activation, evaluated exactly as the
// survivors' scores are (activate_rt), is at most B less eight units in the last place: the hardware's exp and reciprocal are
// good to about one such unit each, so no rounding wobble of theirs can lift a lower z to B.  Where the activation is flat at
// B (a ReLU's zero, a saturated sigmoid) the result falls to the start of the flat part or to -inf: everything that ties is
// admitted.  Supported: sigmoid, tanh, ReLU, leaky ReLU with a positive slope, linear.
__device__ __forceinline__ float preactivation_bound(uint32_t key, uint32_t act, float slope, float alpha, float lambda)
{
    if (key == 0) return -__builtin_inff();   // no bound yet: fewer than k scores seen
    const float B = key_score(key);
    if (act == DSX_ACT_LINEAR) return B;
    const float target = B - fabsf(B) * 1e-6f - 1e-37f;
    float z;
    switch (act) {
    case DSX_ACT_SIGMOID:
        if (target <= 0.0f) return -__builtin_inff();
        z = (target < 1.0f) ? logf(target / (1.0f - target)) : 20.0f;
        break;
    case DSX_ACT_TANH:
        if (target <= -1.0f) return -__builtin_inff();
        z = (target < 1.0f) ? 0.5f * logf((1.0f + target) / (1.0f - target)) : 10.0f;
        break;
    case DSX_ACT_RELU:
        if (target < 0.0f) return -__builtin_inff();
        z = target;
        break;
    case DSX_ACT_LRELU:
        z = (target > 0.0f) ? target : target / slope;
        break;
    default: return -__builtin_inff();
    }
    float delta = fmaxf(fabsf(z), 1.0f) * 9.5367431640625e-7f;   // 2^-20
    for (int it = 0; it < 64; it++) {
        if (activate_rt(z, act, slope, alpha, lambda) <= target) return z;
        z -= delta;
        delta *= 2.0f;
    }
    return -__builtin_inff();
}

// The epilogue below needs the admission bounds of the tile's rows.  Lane t < 32*MI*WM asks for row t's bound here, at the start
// of the kernel: asked for in the epilogue, the load's latency would sit at the end of every tile.
template <int MI, int WM = 2>
__device__ __forceinline__ uint32_t candidate_bound_prefetch(const CandArgs& c, uint32_t row0, uint32_t batch, int tid)
{
    uint32_t key = 0xffffffffu;   // rows beyond the batch admit nothing
    if (tid < 32 * MI * WM && row0 + tid < batch) key = c.row_bound[row0 + tid];
    return key;
}

// Epilogue of a workgroup of WM x WN wavefronts whose wavefront (wm, wn) holds MI x NI accumulators of 32 x 32 (register v of
// lane l: row 8*(v/4) + 4*(l/32) + v%4, column l%32): the tile is only compared with the rows' admission bounds.  A bound is the key
// of a score that k items seen earlier reach, so a lane usually ends after its MI * NI * 16 compares.  The bounds of the
// tile's 32*MI*WM rows are staged in LDS as floats (`lds`: kCandLdsBytes of workgroup memory that is free by now), four
// consecutive rows per 128-bit read; "x >= bound" as floats lets a few scores through whose key is below the bound's (-0.0
// against +0.0), which the merge of the lists sorts out, and keeps NaN scores out, as the scanning top-K does.  A wavefront with survivors first gathers them in a list in LDS and
// then appends the whole list to the rows' global lists, one atomic per survivor but all of them in flight together: asked
// for one by one, each atomic's round trip (thousands of cycles) would be waited for separately.
// bound_key is what candidate_bound_prefetch returned to this lane.  Every lane of the workgroup must call this.
constexpr int kCandWaveList = 256;   // survivors a wavefront gathers before it appends them
template <int MI, int WM = 2, int WN = 2> constexpr int kCandLdsBytes = 32 * MI * WM * 4 + WM * WN * kCandWaveList * 12;

template <int MI, int NI, int WM = 2, int WN = 2, bool PRE = false>
__device__ __forceinline__ void candidate_epilogue(const floatx16 (&acc)[MI][NI], float* lds, const CandArgs& c, uint32_t bound_key,
                                                   uint32_t row0, uint32_t col0, uint32_t batch, uint32_t n, int tid, int wm, int wn, int l32,
                                                   int lhi)
{
    constexpr int BM = 32 * MI * WM;   // at most as many rows as the workgroup has lanes
    float* sBound = lds;
    // key 0: no bound yet (fewer than k items seen), every score that is a number is admitted
    if (tid < BM) {
        float bound = __builtin_inff();   // rows beyond the batch admit nothing
        if (row0 + tid < batch) {
            if constexpr (PRE) bound = preactivation_bound(bound_key, c.act, c.slope, c.alpha, c.lambda);
            else bound = bound_key ? key_score(bound_key) : -__builtin_inff();
        }
        sBound[tid] = bound;
    }
    __syncthreads();
    float bf[MI][4][4];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const float4 t = *reinterpret_cast<const float4*>(&sBound[wm * 32 * MI + i * 32 + 8 * g + 4 * lhi]);
            bf[i][g][0] = t.x; bf[i][g][1] = t.y; bf[i][g][2] = t.z; bf[i][g][3] = t.w;
        }
    // one compare per score, its wavefront-wide result (a scalar register pair) gathered per 32 x 32 block: nothing else
    // happens for a block without survivors
    uint64_t block_mask[MI][NI];
    uint64_t any_mask = 0;
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++) {
            uint64_t m = 0;
#pragma unroll
            for (int v = 0; v < 16; v++) m |= __builtin_amdgcn_ballot_w64(acc[i][j][v] >= bf[i][v / 4][v % 4]);
            block_mask[i][j] = m;
            any_mask |= m;
        }
    if (any_mask == 0) return;   // nothing among this wavefront's scores

    const int wave = tid >> 6, lane = tid & 63;
    uint64_t* sWord = reinterpret_cast<uint64_t*>(lds + BM) + wave * kCandWaveList;
    uint32_t* sRow = reinterpret_cast<uint32_t*>(reinterpret_cast<uint64_t*>(lds + BM) + WM * WN * kCandWaveList) + wave * kCandWaveList;
    uint32_t listed = 0;   // wavefront-uniform
    auto append_all = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        for (uint32_t e = lane; e < listed; e += 64) {
            const uint32_t r = sRow[e];
            const uint64_t word = sWord[e];
            if (r == 0xffffffffu) continue;
            const uint32_t pos = atomicAdd(&c.cand_count[r], 1u);
            if (pos < c.cand_cap)
                c.cand[(uint64_t)r * c.cand_cap + pos] = word;
            else
                *c.overflow = 1u;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        listed = 0;
    };
#pragma unroll
    for (int j = 0; j < NI; j++) {
        const uint32_t col = col0 + wn * 32 * NI + j * 32 + l32;
        const bool col_ok = col < n;   // columns beyond the range hold sums over zero padding, which a bound <= 0 would let through
        const uint64_t col_mask = __builtin_amdgcn_ballot_w64(col_ok);
#pragma unroll
        for (int i = 0; i < MI; i++) {
            if ((block_mask[i][j] & col_mask) == 0) continue;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                float x = acc[i][j][v];
                asm volatile("" : "+v"(x));   // compared afresh: results kept from the pass above would cost more than they save
                const uint64_t mask = __builtin_amdgcn_ballot_w64(x >= bf[i][v / 4][v % 4] && col_ok);
                if (mask == 0) continue;
                const bool cand = (mask >> lane) & 1;
                const uint32_t r = row0 + wm * 32 * MI + i * 32 + 8 * (v / 4) + 4 * lhi + (v % 4);
                const uint32_t count = (uint32_t)__builtin_popcountll(mask);
                if (listed + count > (uint32_t)kCandWaveList) append_all();
                if (cand) {
                    const uint32_t slot = listed + __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
                    float score = x;
                    if constexpr (PRE) score = activate_rt(x, c.act, c.slope, c.alpha, c.lambda);
                    sWord[slot] = ((uint64_t)score_key(score) << 32) | (uint32_t)~(c.col_offset + col);
                    sRow[slot] = (r < batch) ? r : 0xffffffffu;   // (rows beyond the batch have an infinite bound: never taken)
                }
                listed += count;
            }
        }
    }
    append_all();
}

// CalculateActivation (engine/NNLayer.cpp:1646-1683) runs a kernel only for sigmoid, tanh, ReLU, leaky ReLU, ELU, SELU and
// softmax; every other ordinal leaves the unit buffer as it is.  Softmax is a row operation with its own kernel.
inline bool is_elementwise_activation(uint32_t act) { return act != DSX_ACT_SOFTMAX; }

}  // namespace dsx
