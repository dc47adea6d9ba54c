// dsx_knn.hip — device part of the exact KNN search: scores = queries . items^T, then the k best items per query.
//
// The item table is walked in column blocks: each block's scores are produced by the fp32 MFMA GEMM into a scratch
// matrix that stays far smaller than the full [queries x items] product, the block's per-query top-k is taken straight
// from it into packed partial lists, and one merge pass at the end combines the blocks.  A block's k-th score is a lower
// bound of the query's final k-th score, so every later block starts with it as its admission threshold.
#include <algorithm>
#include <hip/hip_runtime.h>
#include "dsx_internal.h"

namespace dsx {

static void* g_knn_ws = nullptr;
static size_t g_knn_ws_bytes = 0;

static uint32_t knn_block_columns(uint32_t rows_padded, uint32_t num_queries)
{
    // about 1 GiB of scores per block, a multiple of 1024 columns
    uint64_t cols = ((uint64_t)1 << 30) / ((uint64_t)std::max(1u, num_queries) * sizeof(float));
    cols = std::max<uint64_t>(1024, cols / 1024 * 1024);
    cols = std::min<uint64_t>(cols, ((uint64_t)rows_padded + 1023) / 1024 * 1024);
    return (uint32_t)cols;
}

static inline size_t align256(size_t x) { return (x + 255) / 256 * 256; }

// a fill kernel rather than hipMemsetAsync: callers may record the search into a HIP graph
__global__ __launch_bounds__(256) void knn_clear_kernel(uint32_t* p, uint32_t n)
{
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0;
}

}  // namespace dsx

using namespace dsx;

extern "C" {

size_t dsx_knn_workspace_bytes(uint32_t rows_padded, uint32_t dim, uint32_t num_queries, uint32_t k)
{
    (void)dim;
    const uint32_t cb = knn_block_columns(rows_padded, num_queries);
    const uint32_t blocks = (rows_padded + cb - 1) / cb;
    return align256((size_t)num_queries * cb * sizeof(float)) + align256((size_t)num_queries * blocks * k * sizeof(uint64_t)) +
           align256((size_t)num_queries * sizeof(uint32_t));
}

int dsx_knn_search(const float* items, uint32_t rows_padded, uint32_t padding, uint32_t dim, const float* queries,
                   uint32_t num_queries, uint32_t k, float* scores, uint32_t* indexes, void* workspace, size_t workspace_bytes,
                   float* elapsed_ms)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(items && queries && scores && indexes, "dsx_knn_search: null device pointer");
    DSX_CHECK_ARG(padding < rows_padded, "dsx_knn_search: padding %u leaves no item of %u", padding, rows_padded);
    DSX_CHECK_ARG(dim > 0, "dsx_knn_search: dim is 0");
    DSX_CHECK_ARG(k >= 1 && k <= 256, "dsx_knn_search: k = %u is outside 1..256", k);
    if (num_queries == 0) return DSX_OK;
    const size_t need = dsx_knn_workspace_bytes(rows_padded, dim, num_queries, k);
    if (workspace) {
        DSX_CHECK_ARG(workspace_bytes >= need, "dsx_knn_search: workspace of %zu bytes, %zu needed", workspace_bytes, need);
    } else {
        if (g_knn_ws_bytes < need) {
            if (g_knn_ws) {
                DSX_HIP(hipStreamSynchronize(ctx().stream));
                DSX_HIP(hipFree(g_knn_ws));
                g_knn_ws = nullptr;
                g_knn_ws_bytes = 0;
            }
            hipError_t e = hipMalloc(&g_knn_ws, need);
            if (e != hipSuccess) return set_error(DSX_ENOMEM, "dsx_knn_search: cannot allocate %zu bytes of workspace: %s", need, hipGetErrorString(e));
            g_knn_ws_bytes = need;
        }
        workspace = g_knn_ws;
    }
    const uint32_t M = rows_padded - padding;
    const uint32_t cb = knn_block_columns(rows_padded, num_queries);
    const uint32_t blocks_alloc = (rows_padded + cb - 1) / cb;
    const uint32_t blocks = (M + cb - 1) / cb;
    float* block_scores = (float*)workspace;
    uint64_t* partial = (uint64_t*)((char*)workspace + align256((size_t)num_queries * cb * sizeof(float)));
    // per query: key of a score that k items of the blocks done so far reach; later blocks admit nothing below it
    uint32_t* row_bound = (uint32_t*)((char*)partial + align256((size_t)num_queries * blocks_alloc * k * sizeof(uint64_t)));
    hipLaunchKernelGGL(knn_clear_kernel, dim3((num_queries + 255) / 256), dim3(256), 0, ctx().stream, row_bound, num_queries);

    hipStream_t s = ctx().stream;
    hipEvent_t ev[3] = {nullptr, nullptr, nullptr};
    float t_gemm = 0.0f, t_topk = 0.0f;
    if (elapsed_ms)
        for (auto& e : ev) DSX_HIP(hipEventCreate(&e));
    int rc = DSX_OK;
    for (uint32_t blk = 0; blk < blocks && rc == DSX_OK; blk++) {
        const uint32_t c0 = blk * cb;
        const uint32_t ncols = std::min(cb, M - c0);
        if (elapsed_ms) hipEventRecord(ev[0], s);
        rc = fc_run(queries, dim, items + c0, rows_padded, 0, nullptr, block_scores, cb, num_queries, dim, ncols, 0, DSX_ACT_LINEAR, nullptr);
        if (rc) break;
        if (elapsed_ms) hipEventRecord(ev[1], s);
        rc = topk_run(block_scores, cb, ncols, num_queries, k, nullptr, nullptr, 0, nullptr, nullptr, nullptr, nullptr, nullptr, c0, partial,
                      blocks, blk, 1, row_bound);
        if (rc) break;
        if (elapsed_ms) {
            hipEventRecord(ev[2], s);
            hipEventSynchronize(ev[2]);
            float a = 0, b = 0;
            hipEventElapsedTime(&a, ev[0], ev[1]);
            hipEventElapsedTime(&b, ev[1], ev[2]);
            t_gemm += a;
            t_topk += b;
        }
    }
    if (rc == DSX_OK) {
        if (elapsed_ms) hipEventRecord(ev[0], s);
        rc = topk_merge(partial, blocks, k, scores, indexes, num_queries);
        if (elapsed_ms && rc == DSX_OK) {
            hipEventRecord(ev[1], s);
            hipEventSynchronize(ev[1]);
            float a = 0;
            hipEventElapsedTime(&a, ev[0], ev[1]);
            t_topk += a;
        }
    }
    if (elapsed_ms) {
        for (auto& e : ev) hipEventDestroy(e);
        elapsed_ms[0] = t_gemm;
        elapsed_ms[1] = t_topk;
    }
    return rc;
}

}  // extern "C"
