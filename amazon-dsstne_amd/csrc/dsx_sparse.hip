// dsx_sparse.hip — input side of a layer: bias initialisation, dense/sparse input loaders and the sparse-Z SpMM.
//
// Sparse Z (the hot one): one 256-lane workgroup per (sample row, column tile).  The row's non-zero column numbers and
// values are staged in LDS in chunks; the 256 lanes are split into G groups of LPR lanes, a group covers one weight row
// with VEC consecutive fp32 columns per lane (128-bit gathers when VEC = 4), and the groups walk the non-zeros interleaved
// (group g takes non-zeros g, g+G, ...), up to sixteen gathers in flight per lane.  The G partial sums are combined through LDS in
// group order, so the result does not depend on scheduling.  Bias and activation can be applied in the same kernel.
#include <type_traits>
#include "dsx_device.h"
#include "dsx_internal.h"

namespace dsx {

constexpr int kSparseThreads = 256;
constexpr int kSparseChunk = 2048;   // non-zeros staged in LDS per pass

// Value of one non-zero as the reference kernels form it: generic T keeps "w * data" converted back to T
// (engine/kernels.cu:828,848), the 8-bit types scale the raw byte by 1/256 (engine/kernels.cu:923,998).
template <typename T> __device__ __forceinline__ float analog_value(float w, T v) { return (float)(T)(w * v); }
template <> __device__ __forceinline__ float analog_value<unsigned char>(float w, unsigned char v) { return w * ((float)v * (float)(1.0 / 256.0)); }
template <> __device__ __forceinline__ float analog_value<signed char>(float w, signed char v) { return w * ((float)v * (float)(1.0 / 256.0)); }

template <int VEC> struct VecT;
template <> struct VecT<4> { using type = float4; };
template <> struct VecT<2> { using type = float2; };
template <> struct VecT<1> { using type = float; };

template <int VEC> __device__ __forceinline__ void load_vec(const float* p, float (&v)[VEC])
{
    if constexpr (VEC == 4) {
        float4 t = *reinterpret_cast<const float4*>(p);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    } else if constexpr (VEC == 2) {
        float2 t = *reinterpret_cast<const float2*>(p);
        v[0] = t.x; v[1] = t.y;
    } else {
        v[0] = *p;
    }
}

template <int VEC> __device__ __forceinline__ void store_vec(float* p, const float (&v)[VEC])
{
    if constexpr (VEC == 4) {
        *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    } else if constexpr (VEC == 2) {
        *reinterpret_cast<float2*>(p) = make_float2(v[0], v[1]);
    } else {
        *p = v[0];
    }
}

// U gathers of one lane in flight (non-zeros t, t+G, ..., t+(U-1)G of the staged chunk), then accumulated in that order.
// Long rows are latency bound on the gather, so the depth of this block sets the time of the longest row.
template <int U, int VEC, bool UNITVAL>
__device__ __forceinline__ void gather_block(const float* wcol, uint32_t stride, const uint32_t* sIdx, const float* sVal, uint32_t t,
                                             uint32_t G, float (&acc)[VEC])
{
    float x[U][VEC];
#pragma unroll
    for (int u = 0; u < U; u++) load_vec<VEC>(wcol + (uint64_t)sIdx[t + u * G] * stride, x[u]);
    if constexpr (UNITVAL) {
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
            for (int v = 0; v < VEC; v++) acc[v] += x[u][v];
    } else {
        float sv[U];
#pragma unroll
        for (int u = 0; u < U; u++) sv[u] = sVal[t + u * G];
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
            for (int v = 0; v < VEC; v++) acc[v] = fmaf(x[u][v], sv[u], acc[v]);
    }
}

struct SparseZArgs {
    uint32_t position, stride;
    const float* weight;
    const uint32_t* index;
    const uint64_t* start;
    const uint64_t* end;
    const uint32_t* sparse_index;
    const float* data_weight;
    const void* sparse_data;
    float* unit;
    float beta;
    const float* bias;   // fused mode only
    uint32_t act;
    float slope, alpha, lambda;
    uint32_t lpr_log2;   // log2 of lanes per weight row
    int tile_major;      // blockIdx.x is the column tile and blockIdx.y the row (see launch_sparse_z); otherwise the other way round
};

// T: storage type of the non-zero values; UNITVAL: every value is exactly 1 (Boolean, unweighted): no multiply;
// FUSED: unit = act(bias + sum) instead of unit = beta * unit + sum.
// DEEP: sixteen gathers per lane in flight (96 registers, five workgroups per CU) — what a launch of many rounds wants, where
// the longest rows set the time; otherwise eight (at most 64 registers, eight workgroups per CU): a launch that then fits the
// GPU in one round does without a second round's start-up.
template <typename T, bool BOOLEAN, bool UNITVAL, int VEC, bool FUSED, bool DEEP>
__global__ __launch_bounds__(kSparseThreads, DEEP ? 4 : 8) void sparse_z_kernel(SparseZArgs a)
{
    __builtin_amdgcn_s_setprio(3);   // short kernels issue ahead of a GEMM's wavefronts that share their SIMD
    __shared__ uint32_t sIdx[kSparseChunk];
    __shared__ float sVal[UNITVAL ? 1 : kSparseChunk];
    __shared__ float sRed[kSparseThreads * VEC];

    const uint32_t b = a.tile_major ? blockIdx.y : blockIdx.x;
    const uint32_t tile = a.tile_major ? blockIdx.x : blockIdx.y;
    uint32_t r = a.position + b;
    if (a.index) r = a.index[r];
    const uint64_t start = a.start[r];
    const uint64_t end = a.end[r];
    const float w = a.data_weight ? a.data_weight[r] : 1.0f;

    const uint32_t lpr = 1u << a.lpr_log2;
    const uint32_t G = kSparseThreads >> a.lpr_log2;
    const uint32_t g = threadIdx.x >> a.lpr_log2;
    const uint32_t lane = threadIdx.x & (lpr - 1);
    const uint32_t col = (tile * lpr + lane) * VEC;
    const bool active = col < a.stride;
    float* urow = a.unit + (uint64_t)b * a.stride;

    if (start >= end) {
        // No non-zeros: the reference's loop body never runs and the unit row keeps what kClearUnit put there.
        if constexpr (FUSED) {
            if (g == 0 && active) {
                float o[VEC];
#pragma unroll
                for (int v = 0; v < VEC; v++) {
                    float x = a.bias ? a.bias[col + v] : 0.0f;
                    o[v] = activate_rt(x, a.act, a.slope, a.alpha, a.lambda);
                }
                store_vec<VEC>(urow + col, o);
            }
        }
        return;
    }

    float acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; v++) acc[v] = 0.0f;
    // (the bias is requested now: asked for after the sums, it would be one more memory round trip at the very end)
    float bz[VEC];
#pragma unroll
    for (int v = 0; v < VEC; v++) bz[v] = 0.0f;
    if constexpr (FUSED) {
        if (g == 0 && active && a.bias) {
#pragma unroll
            for (int v = 0; v < VEC; v++) bz[v] = a.bias[col + v];
        }
    }

    const float* wcol = a.weight + col;
    for (uint64_t cs = start; cs < end; cs += kSparseChunk) {
        const uint32_t n = (uint32_t)min((uint64_t)kSparseChunk, end - cs);
        if (cs != start) __syncthreads();
        for (uint32_t t = threadIdx.x; t < n; t += kSparseThreads) {
            sIdx[t] = a.sparse_index[cs + t];
            if constexpr (!UNITVAL) {
                if constexpr (BOOLEAN)
                    sVal[t] = w;
                else
                    sVal[t] = analog_value<T>(w, reinterpret_cast<const T*>(a.sparse_data)[cs + t]);
            }
        }
        __syncthreads();
        if (active) {
            uint32_t t = g;
            constexpr int U = DEEP ? 16 : 8;
            for (; t + (U - 1) * G < n; t += U * G) gather_block<U, VEC, UNITVAL>(wcol, a.stride, sIdx, sVal, t, G, acc);
            for (; t + 3 * G < n; t += 4 * G) gather_block<4, VEC, UNITVAL>(wcol, a.stride, sIdx, sVal, t, G, acc);
            for (; t < n; t += G) gather_block<1, VEC, UNITVAL>(wcol, a.stride, sIdx, sVal, t, G, acc);
        }
    }

    // Combine the G partial sums in group order.
    if (G > 1) {
#pragma unroll
        for (int v = 0; v < VEC; v++) sRed[(g * lpr + lane) * VEC + v] = acc[v];
        __syncthreads();
        if (g == 0) {
            // all partial sums are read at once and added in group order (G is 4, 8 or 16 with 64, 32 or 16 lanes per row)
            auto combine = [&](auto groups_tag) __attribute__((always_inline)) {
                constexpr int GG = decltype(groups_tag)::value;
                float part[GG - 1][VEC];
#pragma unroll
                for (int gg = 1; gg < GG; gg++)
#pragma unroll
                    for (int v = 0; v < VEC; v++) part[gg - 1][v] = sRed[(gg * lpr + lane) * VEC + v];
#pragma unroll
                for (int gg = 1; gg < GG; gg++)
#pragma unroll
                    for (int v = 0; v < VEC; v++) acc[v] += part[gg - 1][v];
            };
            if (G == 16) combine(std::integral_constant<int, 16>());
            else if (G == 8) combine(std::integral_constant<int, 8>());
            else if (G == 4) combine(std::integral_constant<int, 4>());
            else {
                for (uint32_t gg = 1; gg < G; gg++) {
#pragma unroll
                    for (int v = 0; v < VEC; v++) acc[v] += sRed[(gg * lpr + lane) * VEC + v];
                }
            }
        }
    }
    if (g == 0 && active) {
        float o[VEC];
        if constexpr (FUSED) {
#pragma unroll
            for (int v = 0; v < VEC; v++) {
                float x = bz[v] + acc[v];
                o[v] = activate_rt(x, a.act, a.slope, a.alpha, a.lambda);
            }
        } else {
            if (a.beta == 0.0f) {
#pragma unroll
                for (int v = 0; v < VEC; v++) o[v] = acc[v];
            } else {
                float u[VEC];
                load_vec<VEC>(urow + col, u);
#pragma unroll
                for (int v = 0; v < VEC; v++) o[v] = fmaf(a.beta, u[v], acc[v]);
            }
        }
        store_vec<VEC>(urow + col, o);
    }
}

template <typename T, bool BOOLEAN, bool UNITVAL, bool FUSED>
static int launch_sparse_z(const SparseZArgs& a0, uint32_t batch)
{
    SparseZArgs a = a0;
    // Vector width: 128-bit gathers need the weight rows (and the unit rows) 16-byte aligned.
    auto aligned = [&](int bytes) {
        bool ok = ((uintptr_t)a.weight % bytes == 0) && ((uintptr_t)a.unit % bytes == 0) && (((uint64_t)a.stride * 4) % bytes == 0);
        return ok;
    };
    int vec = aligned(16) ? 4 : (aligned(8) ? 2 : 1);
    uint32_t lanes_needed = (a.stride + vec - 1) / vec;
    // Lanes per weight row: at least 16, at most 64, and half a row where that allows it.  The layer is cut into column tiles
    // that wide (up to 256 columns with 128-bit gathers), each with a workgroup of its own per row whose lane groups share
    // the row's non-zeros; the tile is the fastest grid dimension, so consecutive workgroups — which go to consecutive XCDs —
    // are different tiles of one row, and an XCD's L2 sees some column tiles of the weight matrix instead of all of it
    // (27,278 x 1,024 at batch 4,096: 38 % of the gathers hit in L2 with one tile, 270 -> 163 us with four;
    // 27,278 x 128 at batch 1,024: 14.6 -> 12.1 us with two).
    uint32_t lpr_log2 = 4;
    while ((2u << lpr_log2) < lanes_needed && lpr_log2 < 6) lpr_log2++;
    a.lpr_log2 = lpr_log2;
    uint32_t tiles = (lanes_needed + (1u << lpr_log2) - 1) >> lpr_log2;
    a.tile_major = batch <= 65535;   // (the second grid dimension ends there)
    dim3 grid = a.tile_major ? dim3(tiles, batch) : dim3(batch, tiles);
    hipStream_t s = ctx().stream;
    // (values that are not all 1 need registers for the values as well: only the deep form)
    const bool deep = !UNITVAL || (uint64_t)tiles * batch > 8ull * (uint64_t)ctx().num_cus;   // more than one round of eight workgroups per CU
#define DSX_SPARSE_CASE(V)                                                                                                            \
    case V:                                                                                                                           \
        if constexpr (UNITVAL) {                                                                                                      \
            if (!deep) {                                                                                                              \
                hipLaunchKernelGGL((sparse_z_kernel<T, BOOLEAN, UNITVAL, V, FUSED, false>), grid, dim3(kSparseThreads), 0, s, a);     \
                break;                                                                                                                \
            }                                                                                                                         \
        }                                                                                                                             \
        hipLaunchKernelGGL((sparse_z_kernel<T, BOOLEAN, UNITVAL, V, FUSED, true>), grid, dim3(kSparseThreads), 0, s, a);              \
        break;
    switch (vec) {
        DSX_SPARSE_CASE(4)
        DSX_SPARSE_CASE(2)
        DSX_SPARSE_CASE(1)
    }
#undef DSX_SPARSE_CASE
    DSX_LAUNCH_CHECK("sparse_z_kernel");
    return DSX_OK;
}

template <bool FUSED>
static int dispatch_sparse_z(uint32_t attributes, uint32_t data_type, const SparseZArgs& a, uint32_t batch)
{
    if (attributes & DSX_ATTR_BOOLEAN) {
        if (a.data_weight) return launch_sparse_z<float, true, false, FUSED>(a, batch);
        return launch_sparse_z<float, true, true, FUSED>(a, batch);
    }
    switch (data_type) {
    case DSX_T_UINT: return launch_sparse_z<uint32_t, false, false, FUSED>(a, batch);
    case DSX_T_INT: return launch_sparse_z<int32_t, false, false, FUSED>(a, batch);
    case DSX_T_LLINT: return launch_sparse_z<int64_t, false, false, FUSED>(a, batch);
    case DSX_T_ULLINT: return launch_sparse_z<uint64_t, false, false, FUSED>(a, batch);
    case DSX_T_FLOAT: return launch_sparse_z<float, false, false, FUSED>(a, batch);
    case DSX_T_DOUBLE: return launch_sparse_z<double, false, false, FUSED>(a, batch);
    case DSX_T_UCHAR: return launch_sparse_z<unsigned char, false, false, FUSED>(a, batch);
    case DSX_T_CHAR: return launch_sparse_z<signed char, false, false, FUSED>(a, batch);
    default: return set_error(DSX_EUNSUPPORTED, "sparse Z: data type %u has no sparse kernel", data_type);
    }
}

static int check_sparse_args(const char* fn, uint32_t attributes, uint32_t batch, uint32_t stride, const float* weight,
                             const uint32_t* index, const uint64_t* start, const uint64_t* end, const uint32_t* sparse_index,
                             const float* data_weight, const void* sparse_data, const float* unit)
{
    DSX_CHECK_ARG(stride > 0, "%s: stride is 0", fn);
    DSX_CHECK_ARG(weight && start && end && sparse_index && unit, "%s: null device pointer", fn);
    DSX_CHECK_ARG(!(attributes & DSX_ATTR_INDEXED) || index, "%s: indexed dataset without an index array", fn);
    DSX_CHECK_ARG(!(attributes & DSX_ATTR_WEIGHTED) || data_weight, "%s: weighted dataset without data weights", fn);
    DSX_CHECK_ARG((attributes & DSX_ATTR_BOOLEAN) || sparse_data, "%s: analog dataset without sparse data", fn);
    DSX_CHECK_ARG(batch <= 0x7fffffffu / 1u, "%s: batch too large", fn);
    return DSX_OK;
}

// ---------------------------------------------------------------------------------------------------------------------
// Small elementwise kernels

__global__ __launch_bounds__(256) void clear_unit_kernel(float* unit, const float* b0, const float* b1, const float* b2,
                                                         const float* b3, uint32_t nbias, uint32_t stride, uint64_t size)
{
    uint64_t pos = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t step = (uint64_t)gridDim.x * blockDim.x;
    for (; pos < size; pos += step) {
        uint32_t j = (uint32_t)(pos % stride);
        float s = 0.0f;
        if (nbias > 0) s = b0[j];
        if (nbias > 1) s += b1[j];
        if (nbias > 2) s += b2[j];
        if (nbias > 3) s += b3[j];
        unit[pos] = s;
    }
}

template <typename T> __device__ __forceinline__ float dense_value(T v) { return (float)v; }
// engine/kernels.cu:463 and :476
template <> __device__ __forceinline__ float dense_value<unsigned char>(unsigned char v) { return (float)v * (float)(1.0 / 256.0) - 0.5f; }
template <> __device__ __forceinline__ float dense_value<signed char>(signed char v) { return (float)v * (float)(1.0 / 128.0); }

template <typename T>
__global__ __launch_bounds__(256) void load_input_unit_kernel(uint32_t position, uint32_t stride, float* unit, const uint32_t* index,
                                                              const T* data)
{
    uint32_t r = position + blockIdx.x;
    if (index) r = index[r];
    const T* src = data + (uint64_t)r * stride;
    float* dst = unit + (uint64_t)blockIdx.x * stride;
    for (uint32_t j = blockIdx.y * blockDim.x + threadIdx.x; j < stride; j += gridDim.y * blockDim.x) dst[j] = dense_value<T>(src[j]);
}

template <typename T, bool BOOLEAN>
__global__ __launch_bounds__(256) void scatter_sparse_input_kernel(uint32_t position, uint32_t batch, uint32_t stride, float* unit,
                                                                   const uint32_t* index, const uint64_t* start, const uint64_t* end,
                                                                   const uint32_t* sparse_index, const float* data_weight,
                                                                   const T* sparse_data)
{
    // one wavefront per row; the row has been zero-filled beforehand
    const uint32_t b = (blockIdx.x * blockDim.x + threadIdx.x) / kWave;
    if (b >= batch) return;
    uint32_t r = position + b;
    if (index) r = index[r];
    const float w = data_weight ? data_weight[r] : 1.0f;
    float* dst = unit + (uint64_t)b * stride;
    const uint64_t e = end[r];
    for (uint64_t t = start[r] + (threadIdx.x & (kWave - 1)); t < e; t += kWave) {
        if constexpr (BOOLEAN)
            dst[sparse_index[t]] = w;
        else
            dst[sparse_index[t]] = w * sparse_data[t];   // engine/kernels.cu:215-234: no 8-bit rescaling in this loader
    }
}

__global__ __launch_bounds__(256) void add_buffers_kernel(float* dst, const float* src, uint64_t size)
{
    uint64_t pos = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t step = (uint64_t)gridDim.x * blockDim.x;
    for (; pos < size; pos += step) dst[pos] += src[pos];
}

static inline uint32_t grid_for(uint64_t size, uint32_t threads, uint32_t per_thread = 1)
{
    uint64_t blocks = (size + (uint64_t)threads * per_thread - 1) / ((uint64_t)threads * per_thread);
    uint64_t cap = (uint64_t)ctx().num_cus * 32;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return (uint32_t)blocks;
}

}  // namespace dsx

using namespace dsx;

extern "C" {

int dsx_clear_unit(float* unit, const float* bias0, const float* bias1, const float* bias2, const float* bias3, uint32_t nbias,
                   uint32_t stride, uint32_t batch)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(unit && stride > 0, "dsx_clear_unit: null unit or zero stride");
    DSX_CHECK_ARG(nbias <= 4, "dsx_clear_unit: at most 4 incoming bias vectors (got %u)", nbias);
    const float* bs[4] = {bias0, bias1, bias2, bias3};
    for (uint32_t i = 0; i < nbias; i++) DSX_CHECK_ARG(bs[i], "dsx_clear_unit: bias %u is null", i);
    uint64_t size = (uint64_t)stride * batch;
    if (size == 0) return DSX_OK;
    hipLaunchKernelGGL(clear_unit_kernel, dim3(grid_for(size, 256, 4)), dim3(256), 0, ctx().stream, unit, bias0, bias1, bias2, bias3,
                       nbias, stride, size);
    DSX_LAUNCH_CHECK("clear_unit_kernel");
    return DSX_OK;
}

int dsx_load_input_unit(uint32_t data_type, uint32_t position, uint32_t batch, uint32_t stride, float* unit, const uint32_t* index,
                        const void* data)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(unit && data && stride > 0, "dsx_load_input_unit: null pointer or zero stride");
    if (batch == 0) return DSX_OK;
    dim3 grid(batch, (stride + 1023) / 1024);
    hipStream_t s = ctx().stream;
#define DSX_CASE(tag, T)                                                                                                          \
    case tag: hipLaunchKernelGGL(load_input_unit_kernel<T>, grid, dim3(256), 0, s, position, stride, unit, index, (const T*)data); break;
    switch (data_type) {
        DSX_CASE(DSX_T_UINT, uint32_t)
        DSX_CASE(DSX_T_INT, int32_t)
        DSX_CASE(DSX_T_LLINT, int64_t)
        DSX_CASE(DSX_T_ULLINT, uint64_t)
        DSX_CASE(DSX_T_FLOAT, float)
        DSX_CASE(DSX_T_DOUBLE, double)
        DSX_CASE(DSX_T_UCHAR, unsigned char)
        DSX_CASE(DSX_T_CHAR, signed char)
    default: return set_error(DSX_EUNSUPPORTED, "dsx_load_input_unit: data type %u has no loader", data_type);
    }
#undef DSX_CASE
    DSX_LAUNCH_CHECK("load_input_unit_kernel");
    return DSX_OK;
}

int dsx_load_sparse_input_unit(uint32_t attributes, uint32_t data_type, uint32_t position, uint32_t batch, uint32_t stride,
                               float* unit, const uint32_t* index, const uint64_t* sparse_start, const uint64_t* sparse_end,
                               const uint32_t* sparse_index, const float* data_weight, const void* sparse_data)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(unit && sparse_start && sparse_end && sparse_index && stride > 0, "dsx_load_sparse_input_unit: null pointer or zero stride");
    DSX_CHECK_ARG((attributes & DSX_ATTR_BOOLEAN) || sparse_data, "dsx_load_sparse_input_unit: analog dataset without sparse data");
    if (batch == 0) return DSX_OK;
    if (!(attributes & DSX_ATTR_INDEXED)) index = nullptr;
    if (!(attributes & DSX_ATTR_WEIGHTED)) data_weight = nullptr;
    hipStream_t s = ctx().stream;
    // zero fill by kernel rather than hipMemsetAsync (memset nodes of a captured graph are not trusted on this hardware pool)
    uint64_t size = (uint64_t)batch * stride;
    hipLaunchKernelGGL(clear_unit_kernel, dim3(grid_for(size, 256, 4)), dim3(256), 0, s, unit, nullptr, nullptr, nullptr, nullptr, 0u,
                       stride, size);
    DSX_LAUNCH_CHECK("clear_unit_kernel");
    dim3 grid((batch * kWave + 255) / 256);
#define DSX_CASE(tag, T)                                                                                                         \
    case tag:                                                                                                                    \
        hipLaunchKernelGGL((scatter_sparse_input_kernel<T, false>), grid, dim3(256), 0, s, position, batch, stride, unit, index, \
                           sparse_start, sparse_end, sparse_index, data_weight, (const T*)sparse_data);                          \
        break;
    if (attributes & DSX_ATTR_BOOLEAN) {
        hipLaunchKernelGGL((scatter_sparse_input_kernel<float, true>), grid, dim3(256), 0, s, position, batch, stride, unit, index,
                           sparse_start, sparse_end, sparse_index, data_weight, (const float*)nullptr);
    } else {
        switch (data_type) {
            DSX_CASE(DSX_T_UINT, uint32_t)
            DSX_CASE(DSX_T_INT, int32_t)
            DSX_CASE(DSX_T_LLINT, int64_t)
            DSX_CASE(DSX_T_ULLINT, uint64_t)
            DSX_CASE(DSX_T_FLOAT, float)
            DSX_CASE(DSX_T_DOUBLE, double)
            DSX_CASE(DSX_T_UCHAR, unsigned char)
            DSX_CASE(DSX_T_CHAR, signed char)
        default: return set_error(DSX_EUNSUPPORTED, "dsx_load_sparse_input_unit: data type %u has no loader", data_type);
        }
    }
#undef DSX_CASE
    DSX_LAUNCH_CHECK("scatter_sparse_input_kernel");
    return DSX_OK;
}

int dsx_sparse_z(uint32_t attributes, uint32_t data_type, uint32_t position, uint32_t batch, uint32_t stride, const float* weight,
                 const uint32_t* index, const uint64_t* sparse_start, const uint64_t* sparse_end, const uint32_t* sparse_index,
                 const float* data_weight, const void* sparse_data, float* unit, float beta)
{
    DSX_REQUIRE_INIT();
    int rc = check_sparse_args("dsx_sparse_z", attributes, batch, stride, weight, index, sparse_start, sparse_end, sparse_index,
                               data_weight, sparse_data, unit);
    if (rc) return rc;
    if (batch == 0) return DSX_OK;
    SparseZArgs a{};
    a.position = position;
    a.stride = stride;
    a.weight = weight;
    a.index = (attributes & DSX_ATTR_INDEXED) ? index : nullptr;
    a.start = sparse_start;
    a.end = sparse_end;
    a.sparse_index = sparse_index;
    a.data_weight = (attributes & DSX_ATTR_WEIGHTED) ? data_weight : nullptr;
    a.sparse_data = sparse_data;
    a.unit = unit;
    a.beta = beta;
    return dispatch_sparse_z<false>(attributes, data_type, a, batch);
}

int dsx_sparse_layer_forward(uint32_t attributes, uint32_t data_type, uint32_t position, uint32_t batch, uint32_t stride,
                             const float* weight, const uint32_t* index, const uint64_t* sparse_start, const uint64_t* sparse_end,
                             const uint32_t* sparse_index, const float* data_weight, const void* sparse_data, const float* bias,
                             uint32_t activation, const dsx_act_params* params, float* unit)
{
    DSX_REQUIRE_INIT();
    int rc = check_sparse_args("dsx_sparse_layer_forward", attributes, batch, stride, weight, index, sparse_start, sparse_end,
                               sparse_index, data_weight, sparse_data, unit);
    if (rc) return rc;
    DSX_CHECK_ARG(is_elementwise_activation(activation), "dsx_sparse_layer_forward: activation %u is a row operation; use dsx_sparse_z + dsx_activation", activation);
    if (batch == 0) return DSX_OK;
    SparseZArgs a{};
    a.position = position;
    a.stride = stride;
    a.weight = weight;
    a.index = (attributes & DSX_ATTR_INDEXED) ? index : nullptr;
    a.start = sparse_start;
    a.end = sparse_end;
    a.sparse_index = sparse_index;
    a.data_weight = (attributes & DSX_ATTR_WEIGHTED) ? data_weight : nullptr;
    a.sparse_data = sparse_data;
    a.unit = unit;
    a.beta = 0.0f;
    a.bias = bias;
    a.act = activation;
    a.slope = params ? params->slope : 0.01f;
    a.alpha = params ? params->alpha : 1.0f;
    a.lambda = params ? params->lambda : 1.0f;
    return dispatch_sparse_z<true>(attributes, data_type, a, batch);
}

int dsx_add_buffers(float* dst, const float* src, uint64_t size)
{
    DSX_REQUIRE_INIT();
    if (size == 0) return DSX_OK;
    DSX_CHECK_ARG(dst && src, "dsx_add_buffers: null pointer");
    hipLaunchKernelGGL(add_buffers_kernel, dim3(grid_for(size, 256, 4)), dim3(256), 0, ctx().stream, dst, src, size);
    DSX_LAUNCH_CHECK("add_buffers_kernel");
    return DSX_OK;
}

}  // extern "C"
