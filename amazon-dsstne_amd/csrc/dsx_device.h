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

// CalculateActivation (engine/NNLayer.cpp:1646-1683) runs a kernel only for sigmoid, tanh, ReLU, leaky ReLU, ELU, SELU and
// softmax; every other ordinal leaves the unit buffer as it is.  Softmax is a row operation with its own kernel.
inline bool is_elementwise_activation(uint32_t act) { return act != DSX_ACT_SOFTMAX; }

}  // namespace dsx
