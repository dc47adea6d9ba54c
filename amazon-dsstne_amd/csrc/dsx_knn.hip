// dsx_knn.hip — device part of the exact KNN search: scores = queries . items^T, then the k best items per query.
//
// The first column block of the item table goes through the fp32 MFMA GEMM into a scratch score matrix and the scanning
// top-K; its k-th score per query is a lower bound of the query's final k-th score.  From there on the score matrix is never
// written: the same GEMM kernel runs in candidate mode, where a tile is only compared with the rows' bounds and the few
// scores that reach them are appended to per-query candidate lists.  After every column range (each four times as wide as
// everything before it, so that a range leaves about 4 k candidates per query) a small kernel folds the candidates into
// the query's best list and raises its bound.  Results are exact for any input: a list that fills up (items sorted by
// score, say) raises a flag that the host reads at the end, and the search is then redone block by block — GEMM into the
// scratch matrix, scanning top-K into packed partial lists with the running bound, one merge — which is also the path
// taken while the stream is being captured into a graph (no host read-back there; the caller then passes its own workspace,
// the library's would have to be allocated inside the capture) and for operands that are not 16-byte aligned.  With fp16 storage (dsx_knn_search_f16) the scores come from the f16 MFMA kernel of dsx_knn_f16.hip instead, through
// the same three steps.
#include <algorithm>
#include <hip/hip_runtime.h>
#include "dsx_device.h"
#include "dsx_internal.h"

namespace dsx {

static LibScratch g_knn_ws_of[DSX_MAX_LANES];   // per lane

static int g_knn_last_path = 0;            // how the last search ran: DSX_KNN_PATH_*

static uint32_t knn_block_columns(uint32_t rows_padded, uint32_t num_queries)
{
    // about 1 GiB of scores per block, a multiple of 1024 columns
    uint64_t cols = ((uint64_t)1 << 30) / ((uint64_t)std::max(1u, num_queries) * sizeof(float));
    if (ctx().knobs.knn_block_columns) cols = ctx().knobs.knn_block_columns;
    cols = std::max<uint64_t>(1024, cols / 1024 * 1024);
    cols = std::min<uint64_t>(cols, ((uint64_t)rows_padded + 1023) / 1024 * 1024);
    return (uint32_t)cols;
}

static inline size_t align256(size_t x) { return (x + 255) / 256 * 256; }

// a fill kernel rather than hipMemsetAsync (memset nodes of a captured graph are not trusted on this hardware pool)
__global__ __launch_bounds__(256) void knn_clear_kernel(uint32_t* p, uint32_t n)
{
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0;
}

constexpr uint32_t kCandCap = 4096;   // candidate words per query and column range

struct KnnWorkspace {
    float* block_scores;
    uint64_t* partial;      // block path: [queries][blocks][k]; candidate path: [queries][k], the best lists
    uint32_t* row_bound;    // [queries] key of a score that k items seen so far reach; later columns admit nothing below it
    uint32_t* cand_count;   // [queries]
    uint32_t* overflow;     // [1] (+ padding)
    uint64_t* cand;         // [queries][kCandCap]
    void* queries16;        // fp16 storage: the query batch, [queries rounded up to 256][ld] halves; split products: its bf16 planes
    uint64_t* seg;          // fp16 storage only: [queries][chunks][kCandCap / chunks], the lists of a sweep (knn_f16_sweep_run)
    uint32_t* seg_count;    // fp16 storage only: [queries][64]
    size_t bytes;
};

static KnnWorkspace knn_layout(void* base, uint32_t rows_padded, uint32_t num_queries, uint32_t k, bool f16 = false, uint32_t dim = 0,
                               bool split = false)
{
    const uint32_t cb = knn_block_columns(rows_padded, num_queries);
    const uint32_t blocks = (rows_padded + cb - 1) / cb;
    KnnWorkspace w;
    char* p = (char*)base;
    w.block_scores = (float*)p;
    p += align256((size_t)num_queries * cb * sizeof(float));
    w.partial = (uint64_t*)p;
    p += align256((size_t)num_queries * blocks * k * sizeof(uint64_t));
    w.row_bound = (uint32_t*)p;             // row_bound, cand_count and overflow are cleared together
    w.cand_count = w.row_bound + num_queries;
    w.overflow = w.cand_count + num_queries;
    p += align256(((size_t)2 * num_queries + 64) * sizeof(uint32_t));
    w.cand = (uint64_t*)p;
    p += align256((size_t)num_queries * kCandCap * sizeof(uint64_t));
    w.queries16 = p;
    w.seg = nullptr;
    w.seg_count = nullptr;
    if (f16) {
        p += align256((size_t)knn_f16_rows(num_queries) * knn_f16_ld(dim) * 2);
        w.seg = (uint64_t*)p;
        p += align256((size_t)num_queries * kCandCap * sizeof(uint64_t));
        w.seg_count = (uint32_t*)p;
        p += align256((size_t)num_queries * 64 * sizeof(uint32_t));
    }
    if (split) p += align256((size_t)split_plane_bytes(num_queries, dim));
    w.bytes = (size_t)(p - (char*)base);
    return w;
}

// Where the scores of a column range come from: the fp32 table through fc_gemm_kernel, or the fp16 table through knn_f16_kernel.
struct KnnOperands {
    bool f16 = false;
    bool split = false;                 // fp32 products from bf16 matrix instructions: item_planes / query_planes (dsx_fc_split)
    const void* item_planes = nullptr;
    const void* query_planes = nullptr;
    const float* items = nullptr;       // fp32: column-major [dim][rows_padded]
    const float* queries = nullptr;     // fp32: [queries][dim]
    const char* items16 = nullptr;      // fp16: [rows rounded up to 256][ld]
    const void* queries16 = nullptr;
    uint32_t rows_padded = 0, dim = 0, ld16 = 0;

    int into_matrix(uint32_t c0, uint32_t ncols, uint32_t num_queries, float* Z, uint32_t ldz) const
    {
        if (f16) return knn_f16_scores_run(queries16, items16 + (uint64_t)c0 * ld16 * 2, ld16, num_queries, ncols, Z, ldz, nullptr);
        if (split)
            return fc_split_run(query_planes, item_planes, split_rows_padded(rows_padded), c0, nullptr, Z, ldz, num_queries, dim, ncols, 0,
                                DSX_ACT_LINEAR, nullptr, nullptr, nullptr);
        return fc_run(queries, dim, items + c0, rows_padded, 0, nullptr, Z, ldz, num_queries, dim, ncols, 0, DSX_ACT_LINEAR, nullptr);
    }
    // *chunks_used: how many (row, chunk) lists of seg the range filled besides the shared lists (0: none)
    int into_candidates(uint32_t c0, uint32_t ncols, uint32_t num_queries, const CandArgs& cand, uint64_t* seg, uint32_t* seg_count,
                        uint32_t* chunks_used) const
    {
        *chunks_used = 0;
        if (f16)
            return knn_f16_candidates_run(queries16, items16 + (uint64_t)c0 * ld16 * 2, ld16, num_queries, ncols, cand, seg, seg_count, kCandCap,
                                          ctx().knobs.knn_f16_sweep, chunks_used);
        if (split) return fc_split_candidates_run(query_planes, item_planes, split_rows_padded(rows_padded), c0, num_queries, dim, ncols, cand);
        return fc_candidates_run(queries, dim, items + c0, rows_padded, num_queries, dim, ncols, cand);
    }
};

struct KnnTimer {
    hipEvent_t ev[2] = {nullptr, nullptr};
    bool on = false;
    float gemm = 0.0f, topk = 0.0f;
    void start(hipStream_t s) { if (on) hipEventRecord(ev[0], s); }
    void stop(hipStream_t s, float& into)
    {
        if (!on) return;
        hipEventRecord(ev[1], s);
        hipEventSynchronize(ev[1]);
        float ms = 0.0f;
        hipEventElapsedTime(&ms, ev[0], ev[1]);
        into += ms;
    }
};

// Block by block through the scratch score matrix; exact for any input, no host read-back.
static int knn_search_blocks(const KnnWorkspace& w, const KnnOperands& op, uint32_t M, uint32_t num_queries, uint32_t k, float* scores,
                             uint32_t* indexes, KnnTimer& t)
{
    hipStream_t s = ctx().stream;
    const uint32_t cb = knn_block_columns(op.rows_padded, num_queries);
    const uint32_t blocks = (M + cb - 1) / cb;
    hipLaunchKernelGGL(knn_clear_kernel, dim3((num_queries + 255) / 256), dim3(256), 0, s, w.row_bound, num_queries);
    for (uint32_t blk = 0; blk < blocks; blk++) {
        const uint32_t c0 = blk * cb;
        const uint32_t ncols = std::min(cb, M - c0);
        t.start(s);
        int rc = op.into_matrix(c0, ncols, num_queries, w.block_scores, cb);
        if (rc) return rc;
        t.stop(s, t.gemm);
        t.start(s);
        rc = topk_run(w.block_scores, cb, ncols, num_queries, k, nullptr, nullptr, 0, nullptr, nullptr, nullptr, nullptr, nullptr, c0,
                      w.partial, blocks, blk, 1, w.row_bound);
        if (rc) return rc;
        t.stop(s, t.topk);
    }
    t.start(s);
    int rc = topk_merge(w.partial, blocks, k, scores, indexes, num_queries);
    t.stop(s, t.topk);
    return rc;
}

// First block as above, the rest in candidate mode.  *overflowed tells the caller to redo the search block by block.
static int knn_search_candidates(const KnnWorkspace& w, const KnnOperands& op, uint32_t M, uint32_t num_queries, uint32_t k, float* scores,
                                 uint32_t* indexes, KnnTimer& t, bool* overflowed)
{
    hipStream_t s = ctx().stream;
    const uint32_t cb = knn_block_columns(op.rows_padded, num_queries);
    const uint32_t clear_words = 2 * num_queries + 64;
    hipLaunchKernelGGL(knn_clear_kernel, dim3((clear_words + 255) / 256), dim3(256), 0, s, w.row_bound, clear_words);
    if (w.seg_count) hipLaunchKernelGGL(knn_clear_kernel, dim3((num_queries * 64 + 255) / 256), dim3(256), 0, s, w.seg_count, num_queries * 64);
    // The first block only has to give every query a usable bound; a quarter of a column block does (measured on 2 M items x 4,096
    // queries: 8 K to 32 K columns are level, the full 64 K cost 0.1 ms more in stores and scan).  A width set by the caller is kept.
    uint32_t done = std::min(cb, M);
    if (!ctx().knobs.knn_block_columns) done = std::min<uint32_t>(done, std::max<uint32_t>(1024, cb / 4 / 1024 * 1024));
    t.start(s);
    int rc = op.into_matrix(0, done, num_queries, w.block_scores, cb);
    if (rc) return rc;
    t.stop(s, t.gemm);
    t.start(s);
    rc = topk_run(w.block_scores, cb, done, num_queries, k, nullptr, nullptr, 0, nullptr, nullptr, nullptr, nullptr, nullptr, 0, w.partial, 1, 0,
                  1, w.row_bound);
    if (rc) return rc;
    t.stop(s, t.topk);
    while (done < M) {
        // a multiple of the tile width keeps every range's first column 16-byte aligned
        const uint32_t ncols = (uint32_t)std::min<uint64_t>((uint64_t)M - done, (uint64_t)done * 4 / 128 * 128);
        t.start(s);
        const CandArgs cand{w.row_bound, w.cand, w.cand_count, kCandCap, done, w.overflow};
        uint32_t chunks = 0;
        rc = op.into_candidates(done, ncols, num_queries, cand, w.seg, w.seg_count, &chunks);
        if (rc) return rc;
        t.stop(s, t.gemm);
        t.start(s);
        rc = knn_refresh(w.partial, w.cand, w.cand_count, kCandCap, k, w.row_bound, num_queries, chunks ? w.seg : nullptr, w.seg_count, chunks,
                         chunks ? kCandCap / chunks : 0);
        if (rc) return rc;
        t.stop(s, t.topk);
        done += ncols;
    }
    t.start(s);
    rc = topk_merge(w.partial, 1, k, scores, indexes, num_queries);
    if (rc) return rc;
    t.stop(s, t.topk);
    uint32_t flag = 0;
    DSX_HIP(hipMemcpyAsync(&flag, w.overflow, sizeof(flag), hipMemcpyDeviceToHost, s));
    DSX_HIP(hipStreamSynchronize(s));
    *overflowed = flag != 0;
    return DSX_OK;
}

}  // namespace dsx

using namespace dsx;

extern "C" {

int dsx_testing_set_knn_block_columns(uint32_t columns)
{
    ctx().knobs.knn_block_columns = columns;
    return DSX_OK;
}

int dsx_knn_last_search_path(void) { return g_knn_last_path; }

int dsx_testing_set_knn_f16_sweep(int mode)
{
    DSX_CHECK_ARG(mode >= 0 && mode <= 3, "dsx_testing_set_knn_f16_sweep: mode %d (0 to 3)", mode);
    ctx().knobs.knn_f16_sweep = mode;
    return DSX_OK;
}

size_t dsx_knn_workspace_bytes(uint32_t rows_padded, uint32_t dim, uint32_t num_queries, uint32_t k)
{
    (void)dim;
    return knn_layout(nullptr, rows_padded, num_queries, k).bytes;
}

size_t dsx_knn_workspace_bytes_f16(uint32_t rows_padded, uint32_t dim, uint32_t num_queries, uint32_t k)
{
    return knn_layout(nullptr, rows_padded, num_queries, k, true, dim).bytes;
}

size_t dsx_knn_workspace_bytes_split(uint32_t rows_padded, uint32_t dim, uint32_t num_queries, uint32_t k)
{
    return knn_layout(nullptr, rows_padded, num_queries, k, false, dim, true).bytes;
}

size_t dsx_knn_f16_table_bytes(uint32_t rows_padded, uint32_t dim) { return (size_t)knn_f16_rows(rows_padded) * knn_f16_ld(dim) * 2; }

int dsx_knn_f16_convert_items(const float* items, uint32_t rows_padded, uint32_t padding, uint32_t dim, void* items_f16)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(items && items_f16, "dsx_knn_f16_convert_items: null device pointer");
    DSX_CHECK_ARG(padding < rows_padded && dim > 0, "dsx_knn_f16_convert_items: rows_padded %u, padding %u, dim %u", rows_padded, padding, dim);
    DSX_CHECK_ARG(((uintptr_t)items_f16 % 16) == 0, "dsx_knn_f16_convert_items: the fp16 table is not 16-byte aligned");
    return knn_to_f16(items, true, rows_padded, rows_padded - padding, dim, items_f16, (uint32_t)knn_f16_rows(rows_padded));
}

}  // extern "C"

// Both precisions: workspace, the two paths, timing.
static int knn_search_common(KnnOperands& op, uint32_t padding, uint32_t num_queries, uint32_t k, float* scores, uint32_t* indexes, void* workspace,
                             size_t workspace_bytes, float* elapsed_ms, bool aligned, const float* queries_f32)
{
    const size_t need = knn_layout(nullptr, op.rows_padded, num_queries, k, op.f16, op.dim, op.split).bytes;
    if (workspace) {
        DSX_CHECK_ARG(workspace_bytes >= need, "dsx_knn_search: workspace of %zu bytes, %zu needed", workspace_bytes, need);
        DSX_CHECK_ARG(((uintptr_t)workspace % 256) == 0, "dsx_knn_search: workspace is not 256-byte aligned");
    } else {
        LibScratch& ws = g_knn_ws_of[current_lane()];
        if (int rc = lib_scratch_reserve(ws, need, "dsx_knn_search workspace")) return rc;
        workspace = ws.ptr;
    }
    const KnnWorkspace w = knn_layout(workspace, op.rows_padded, num_queries, k, op.f16, op.dim, op.split);
    const uint32_t M = op.rows_padded - padding;
    hipStream_t s = ctx().stream;
    KnnTimer t;
    if (elapsed_ms) {
        t.on = true;
        for (auto& e : t.ev) DSX_HIP(hipEventCreate(&e));
    }
    int rc = DSX_OK;
    if (op.f16) {   // the query batch in the table's format (knn/KnnExactGpu.cu:108-116); counted as GEMM time like the copy it replaces
        t.start(s);
        rc = knn_to_f16(queries_f32, false, op.dim, num_queries, op.dim, w.queries16, (uint32_t)knn_f16_rows(num_queries));
        if (rc) return rc;
        t.stop(s, t.gemm);
        op.queries16 = w.queries16;
    }
    if (op.split) {   // the query batch as bf16 planes, counted as GEMM time too
        t.start(s);
        rc = fc_split_planes_run(queries_f32, op.dim, 1, num_queries, op.dim, w.queries16);
        if (rc) return rc;
        t.stop(s, t.gemm);
        op.query_planes = w.queries16;
    }
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    hipStreamIsCapturing(s, &capturing);
    const bool candidates = aligned && capturing == hipStreamCaptureStatusNone && M > knn_block_columns(op.rows_padded, num_queries);
    bool redo = !candidates;
    if (rc == DSX_OK && candidates) rc = knn_search_candidates(w, op, M, num_queries, k, scores, indexes, t, &redo);
    g_knn_last_path = !candidates ? DSX_KNN_PATH_BLOCKS : (redo ? DSX_KNN_PATH_CANDIDATES_REDONE : DSX_KNN_PATH_CANDIDATES);
    if (rc == DSX_OK && redo) rc = knn_search_blocks(w, op, M, num_queries, k, scores, indexes, t);
    if (elapsed_ms) {
        for (auto& e : t.ev) hipEventDestroy(e);
        elapsed_ms[0] = t.gemm;
        elapsed_ms[1] = t.topk;
    }
    return rc;
}

extern "C" {

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
    KnnOperands op;
    op.items = items;
    op.queries = queries;
    op.rows_padded = rows_padded;
    op.dim = dim;
    const bool aligned = ((uintptr_t)items % 16) == 0 && ((uintptr_t)queries % 16) == 0 && (rows_padded % 4) == 0 && (dim % 4) == 0;
    return knn_search_common(op, padding, num_queries, k, scores, indexes, workspace, workspace_bytes, elapsed_ms, aligned, nullptr);
}

int dsx_knn_search_split(const void* item_planes, uint32_t rows_padded, uint32_t padding, uint32_t dim, const float* queries,
                         uint32_t num_queries, uint32_t k, float* scores, uint32_t* indexes, void* workspace, size_t workspace_bytes,
                         float* elapsed_ms)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(item_planes && queries && scores && indexes, "dsx_knn_search_split: null device pointer");
    DSX_CHECK_ARG(((uintptr_t)item_planes % 16) == 0, "dsx_knn_search_split: the item planes are not 16-byte aligned");
    DSX_CHECK_ARG(padding < rows_padded, "dsx_knn_search_split: padding %u leaves no item of %u", padding, rows_padded);
    DSX_CHECK_ARG(dim > 0, "dsx_knn_search_split: dim is 0");
    DSX_CHECK_ARG(k >= 1 && k <= 256, "dsx_knn_search_split: k = %u is outside 1..256", k);
    DSX_CHECK_ARG((uint64_t)split_plane_bytes(rows_padded, dim) / 3 < (1ull << 32), "dsx_knn_search_split: a plane of the item table of 4 GiB or more");
    if (num_queries == 0) return DSX_OK;
    KnnOperands op;
    op.split = true;
    op.item_planes = item_planes;
    op.rows_padded = rows_padded;
    op.dim = dim;
    return knn_search_common(op, padding, num_queries, k, scores, indexes, workspace, workspace_bytes, elapsed_ms, true, queries);
}

int dsx_knn_search_f16(const void* items_f16, uint32_t rows_padded, uint32_t padding, uint32_t dim, const float* queries,
                       uint32_t num_queries, uint32_t k, float* scores, uint32_t* indexes, void* workspace, size_t workspace_bytes,
                       float* elapsed_ms)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(items_f16 && queries && scores && indexes, "dsx_knn_search_f16: null device pointer");
    DSX_CHECK_ARG(((uintptr_t)items_f16 % 16) == 0, "dsx_knn_search_f16: the fp16 table is not 16-byte aligned");
    DSX_CHECK_ARG(padding < rows_padded, "dsx_knn_search_f16: padding %u leaves no item of %u", padding, rows_padded);
    DSX_CHECK_ARG(dim > 0, "dsx_knn_search_f16: dim is 0");
    DSX_CHECK_ARG(k >= 1 && k <= 256, "dsx_knn_search_f16: k = %u is outside 1..256", k);
    if (num_queries == 0) return DSX_OK;
    KnnOperands op;
    op.f16 = true;
    op.items16 = (const char*)items_f16;
    op.rows_padded = rows_padded;
    op.dim = dim;
    op.ld16 = knn_f16_ld(dim);
    return knn_search_common(op, padding, num_queries, k, scores, indexes, workspace, workspace_bytes, elapsed_ms, true, queries);
}

}  // extern "C"
