// dsx_internal.h — shared state and helpers of libdsx_hip.so (not part of the public ABI).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include "dsx.h"
#include "dsx_testing.h"

namespace dsx {

// Switches of include/dsx_testing.h (0 = default unless stated).
struct TestKnobs {
    uint32_t split_tile_rows = 0;
    uint32_t fc_topk_first_columns = 0;
    uint32_t fc_topk_candidate_capacity = 0;
    uint32_t knn_block_columns = 0;
    int knn_f16_sweep = 1;
};

struct Context {
    TestKnobs knobs;
    bool initialized = false;
    bool sync_launches = false;   // DSX_SYNC=1: wait for every kernel right after its launch
    int users = 0;          // dsx_init calls not yet matched by dsx_shutdown
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    int num_cus = 0;
    size_t gpu_bytes = 0;   // bytes currently held through dsx_malloc / dsx_malloc_managed
    size_t cpu_bytes = 0;   // bytes currently held through dsx_malloc_host
};

Context& ctx();

// Device memory the library allocates for itself (split top-K lists, KNN workspace): grown on demand, counted by
// dsx_get_memory_usage, released by dsx_shutdown.
struct LibScratch {
    void* ptr = nullptr;
    size_t bytes = 0;
    bool listed = false;
};
// Makes s hold at least `bytes` (contents are not preserved when it grows; the selected lane is waited for before the old
// block is freed).
int lib_scratch_reserve(LibScratch& s, size_t bytes, const char* what);
// fn runs once in the last dsx_shutdown, before the library's memory is released (file-scope state of the other translation units).
void at_shutdown(void (*fn)());
int current_lane();   // 0 or 1: which of the two in-order streams ctx().stream is (scratch buffers are kept per lane)
int set_error(int code, const char* fmt, ...);
int sync_after_launch(const char* fn, const char* kernel);   // DSX_SYNC=1, see DSX_LAUNCH_CHECK

// engine/NNTypes.h:49
constexpr float kMaxValue = 999999999999999.0f;

}  // namespace dsx

#define DSX_REQUIRE_INIT()                                                                     \
    do {                                                                                       \
        if (!dsx::ctx().initialized) return dsx::set_error(DSX_ENOTINIT, "%s: dsx_init has not been called", __func__); \
    } while (0)

#define DSX_HIP(call)                                                                                          \
    do {                                                                                                       \
        hipError_t e_ = (call);                                                                                \
        if (e_ != hipSuccess) return dsx::set_error(DSX_EHIP, "%s: %s failed: %s", __func__, #call, hipGetErrorString(e_)); \
    } while (0)

#define DSX_CHECK_ARG(cond, ...)                                  \
    do {                                                          \
        if (!(cond)) return dsx::set_error(DSX_EINVAL, __VA_ARGS__); \
    } while (0)

// After a kernel launch: pick up launch-configuration errors (the analogue of LAUNCHERROR, engine/GpuTypes.h:215-223).  With
// DSX_SYNC=1 in the environment when dsx_init runs (the reference's compile-time SYNCHRONOUS, engine/GpuTypes.h:147-176) every
// launch is also waited for, so that a failure inside a kernel is reported by the call that launched it, with the kernel's name;
// never while the stream is being captured into a graph.
#define DSX_LAUNCH_CHECK(name)                                                                                     \
    do {                                                                                                           \
        hipError_t e_ = hipGetLastError();                                                                         \
        if (e_ != hipSuccess) return dsx::set_error(DSX_EHIP, "%s: launch of %s failed: %s", __func__, name, hipGetErrorString(e_)); \
        if (dsx::ctx().sync_launches) {                                                                            \
            if (int rc_ = dsx::sync_after_launch(__func__, name)) return rc_;                                      \
        }                                                                                                          \
    } while (0)

namespace dsx {
// Top-K building blocks shared with the KNN search (dsx_topk.hip).
// topk_run: per-row top-k of in[batch][pitch] over the first `width` columns.  With partial != NULL the packed lists go to
// partial[b][partial_slot0 + segment][k] (forced_segments workgroups per row) instead of keys/values.  With fixed_scratch the
// lists of rows split over segments go there instead of into memory the library allocates; a call whose lists exceed
// fixed_scratch_words fails.
int topk_run(const float* in, uint32_t pitch, uint32_t width, uint32_t batch, uint32_t k, float* keys, uint32_t* values,
             uint32_t position, const uint32_t* index, const uint64_t* fstart, const uint64_t* fend, const uint32_t* fidx,
             const float* fmul, uint32_t col_offset, uint64_t* partial, uint32_t partial_slots, uint32_t partial_slot0,
             uint32_t forced_segments, uint32_t* row_bound = nullptr, uint64_t* fixed_scratch = nullptr,
             size_t fixed_scratch_words = 0);
// Looks up this device's address of the fixed scratch array behind dsx_topk_filtered_static (called by dsx_init with the
// device current).
int topk_static_setup(int device);
int topk_merge(const uint64_t* partial, uint32_t slots, uint32_t k, float* keys, uint32_t* values, uint32_t batch);
// GEMM building block shared with the KNN search (dsx_fc.hip): Z = X.W (+bias, activation), see dsx_fc_forward.
int fc_run(const float* X, uint32_t ldx, const float* W, uint32_t ldw, int transposed, const float* bias, float* Z, uint32_t ldz,
           uint32_t batch, uint32_t k, uint32_t n, int accumulate, uint32_t activation, const dsx_act_params* params,
           float* seg_max = nullptr, uint32_t* seg_width = nullptr, void* out_planes = nullptr);
// Candidate mode of the same kernel (exact KNN): scores are compared with the rows' bounds and the survivors appended to
// per-row lists as packed words (CandArgs); nothing else is written.  knn_refresh folds a row's candidates into its best
// list.  The caller guarantees 16-byte aligned operands with pitches that are multiples of four floats.
struct CandArgs;
// The same products from bf16 matrix instructions (dsx_fc_split / dsx_fc_forward_split): planes of an operand
// (src element (r, kk) = src[r * stride_r + kk * stride_k]), their size and padded row count, the GEMM on a window of columns
// of the W planes (wrows: their padded rows; wcol0: first column, a multiple of 128), and its candidate mode.
uint32_t split_rows_padded(uint32_t rows);
uint64_t split_plane_bytes(uint32_t rows, uint32_t k);
int fc_split_planes_run(const float* src, uint64_t stride_r, uint64_t stride_k, uint32_t rows, uint32_t k, void* planes);
int fc_split_run(const void* Xs, const void* Ws, uint32_t wrows, uint32_t wcol0, const float* bias, float* Z, uint32_t ldz, uint32_t batch,
                 uint32_t k, uint32_t n, int accumulate, uint32_t activation, const dsx_act_params* params, float* seg_max,
                 uint32_t* seg_width);
int fc_split_candidates_run(const void* Xs, const void* Ws, uint32_t wrows, uint32_t wcol0, uint32_t batch, uint32_t k, uint32_t n,
                            const CandArgs& cand, bool layer = false, const float* bias = nullptr);
int fc_candidates_run(const float* X, uint32_t ldx, const float* W, uint32_t ldw, uint32_t batch, uint32_t k, uint32_t n,
                      const CandArgs& cand);
// The same for a layer (pre-activation sums compared with bounds derived from activated scores, bias folded in).
int fc_layer_candidates_run(const float* X, uint32_t ldx, const float* W, uint32_t ldw, const float* bias, uint32_t batch, uint32_t k,
                            uint32_t n, const CandArgs& cand);
// Output layer fused with its top-K (dsx_topk.hip): folds every row's candidates, minus the columns its filter lists, into its
// best list and raises its bound; with keys != NULL (last column range) writes the result instead.  A row whose candidate list
// overflowed is flagged, and recomputed from X, W and bias in the last range's call.
struct LayerRefresh {
    uint64_t* best;
    const uint64_t* cand;
    uint32_t* cand_count;
    uint32_t cap, k;
    uint32_t* row_bound;
    uint32_t* row_flag;
    uint32_t* flagged_total;
    uint32_t position;
    const uint32_t* index;
    const uint64_t* fstart;
    const uint64_t* fend;
    const uint32_t* fidx;
    float* keys;
    uint32_t* values;
    const float* X;
    const float* W;
    const float* bias;
    uint32_t ldx, ldw, kdim, n;
    uint32_t first_columns;   // width of the first block (scanned with the filter applied)
    uint32_t act;
    float slope, alpha, lambda;
};
int layer_refresh_run(const LayerRefresh& r, uint32_t batch);
// fp16 storage of the KNN operands (dsx_knn_f16.hip): padded row-major layout, conversion, and the score kernel in store mode
// (cand == NULL: Z[batch][ldz]) or candidate mode.
uint32_t knn_f16_ld(uint32_t dim);
uint64_t knn_f16_rows(uint64_t rows);
int knn_to_f16(const float* src, bool colmajor, uint64_t src_ld, uint32_t rows_valid, uint32_t dim, void* dst, uint32_t rows_out);
int knn_f16_scores_run(const void* queries16, const void* items16, uint32_t ld, uint32_t batch, uint32_t n, float* Z, uint32_t ldz,
                       const CandArgs* cand);
int knn_refresh(uint64_t* best, const uint64_t* cand, uint32_t* cand_count, uint32_t cap, uint32_t k, uint32_t* row_bound, uint32_t batch,
                const uint64_t* seg = nullptr, uint32_t* seg_count = nullptr, uint32_t chunks = 0, uint32_t seg_cap = 0);
// fp16 storage, candidate mode of a column range: one workgroup per tile, or (long ranges) workgroups that sweep a chunk of the
// range each and keep (row, chunk) lists of their own (seg [queries][chunks][seg_words / chunks], seg_count [queries][64]); full
// lists spill into cand's shared ones.  mode: see dsx_testing_set_knn_f16_sweep.  *chunks_used is what knn_refresh needs to know.
int knn_f16_candidates_run(const void* queries16, const void* items16, uint32_t ld, uint32_t batch, uint32_t n, const CandArgs& cand,
                           uint64_t* seg, uint32_t* seg_count, uint32_t seg_words, int mode, uint32_t* chunks_used);
}  // namespace dsx
