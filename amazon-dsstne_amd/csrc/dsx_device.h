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
};

// Epilogue of a 2 x 2 wavefront workgroup whose wavefront (wm, wn) holds MI x NI accumulators of 32 x 32 (register v of lane l:
// row 8*(v/4) + 4*(l/32) + v%4, column l%32): the tile is only compared with the rows' admission bounds.  A bound is the key
// of a score that k items seen earlier reach, so almost every tile ends after MI * NI * 16 compares per lane; the few
// survivors are appended to their rows' lists with one atomic each.  The bounds of the tile's 64*MI rows are staged in LDS
// (sBound, free for use by now) as floats, four consecutive rows per 128-bit read; a NaN score fails "x < bound" and is
// sorted out by its key.  Every lane of the workgroup must call this.
template <int MI, int NI>
__device__ __forceinline__ void candidate_epilogue(const floatx16 (&acc)[MI][NI], float* sBound, const CandArgs& c, uint32_t row0,
                                                   uint32_t col0, uint32_t batch, uint32_t n, int tid, int wm, int wn, int l32, int lhi)
{
    constexpr int BM = 64 * MI;
    if (tid < BM) {
        const uint32_t r = row0 + tid;
        sBound[tid] = (r < batch) ? key_score(c.row_bound[r]) : __builtin_inff();
    }
    __syncthreads();
    float bf[MI][4][4];
    bool any = false;
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const float4 t = *reinterpret_cast<const float4*>(&sBound[wm * 32 * MI + i * 32 + 8 * g + 4 * lhi]);
            bf[i][g][0] = t.x; bf[i][g][1] = t.y; bf[i][g][2] = t.z; bf[i][g][3] = t.w;
        }
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) any |= !(acc[i][j][v] < bf[i][v / 4][v % 4]);
    if (!any) return;
#pragma unroll
    for (int j = 0; j < NI; j++) {
        const uint32_t col = col0 + wn * 32 * NI + j * 32 + l32;
        if (col >= n) continue;
#pragma unroll
        for (int i = 0; i < MI; i++) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const float x = acc[i][j][v];
                if (x < bf[i][v / 4][v % 4]) continue;
                const uint32_t r = row0 + wm * 32 * MI + i * 32 + 8 * (v / 4) + 4 * lhi + (v % 4);
                if (r >= batch) continue;
                const uint32_t key = score_key(x);
                if (key < c.row_bound[r]) continue;
                const uint32_t pos = atomicAdd(&c.cand_count[r], 1u);
                if (pos < c.cand_cap)
                    c.cand[(uint64_t)r * c.cand_cap + pos] = ((uint64_t)key << 32) | (uint32_t)~(c.col_offset + col);
                else
                    *c.overflow = 1u;
            }
        }
    }
}

// CalculateActivation (engine/NNLayer.cpp:1646-1683) runs a kernel only for sigmoid, tanh, ReLU, leaky ReLU, ELU, SELU and
// softmax; every other ordinal leaves the unit buffer as it is.  Softmax is a row operation with its own kernel.
inline bool is_elementwise_activation(uint32_t act) { return act != DSX_ACT_SOFTMAX; }

}  // namespace dsx
