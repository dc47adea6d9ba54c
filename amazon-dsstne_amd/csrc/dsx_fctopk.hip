// dsx_fctopk.hip — a fully connected output layer and the (filtered) top-K of its result in one call: the [batch x n] result is
// never stored.
//
// The reference runs the output layer into its unit buffer (cublasSgemm + bias + activation, engine/NNLayer.cpp:994-1167), copies
// the buffer to the host, multiplies the sample's own items by 0 there and runs kCalculateTopK over all n columns
// (utils/NNRecsGenerator.cpp:83-150).  Here only the first few thousand columns are produced as a matrix (a scratch block) and
// scanned: that leaves, per row, a best list and the key of its k-th score.  Every later column range, each several times as
// wide as everything before it, runs the same GEMM kernel in candidate mode: the tile's pre-activation sums are compared with
// the rows' bounds in registers and only the few survivors are activated and appended to per-row lists, which a small kernel
// folds into the best lists after dropping the columns the row's filter names (a row whose result a listed column's score * 0
// could enter - fewer than k scores above 0 - is recomputed with those zeros in place).  Exact for any input: admission is a superset
// of "score >= current k-th score" (preactivation_bound in dsx_device.h), lists are merged under the total order (score
// descending, column ascending), and a row whose list fills up is recomputed from scratch on the device.
#include <algorithm>
#include "dsx_device.h"
#include "dsx_internal.h"

namespace dsx {

constexpr uint32_t kLayerCandCap = 4096;       // candidate words per row and column range
static LibScratch g_layer_ws_of[DSX_MAX_LANES];   // per lane
// Pinned host memory: the device stores 1 in a word when it flags a row.  One word per weight matrix (the layer a call belongs
// to), so that one layer's tied scores say nothing about another's; kFlagWords matrices at a time, the oldest gives way.
constexpr int kFlagWords = 64;
static uint32_t* g_layer_flagged = nullptr;
static const void* g_flag_owner[kFlagWords] = {};
static int g_flag_next = 0;

static void layer_flags_release()
{
    if (g_layer_flagged) hipHostFree(g_layer_flagged);
    g_layer_flagged = nullptr;
    for (auto& o : g_flag_owner) o = nullptr;
    g_flag_next = 0;
}

static int layer_flag_slot(const void* W, bool create)
{
    for (int i = 0; i < kFlagWords; i++)
        if (g_flag_owner[i] == W) return i;
    if (!create) return -1;
    const int i = g_flag_next;
    g_flag_next = (g_flag_next + 1) % kFlagWords;
    g_flag_owner[i] = W;
    *(volatile uint32_t*)&g_layer_flagged[i] = 0;
    return i;
}

__global__ __launch_bounds__(256) void layer_clear_kernel(uint32_t* p, uint32_t n)
{
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0;
}

static inline size_t align256(size_t x) { return (x + 255) / 256 * 256; }

static uint32_t layer_first_columns(uint32_t n, uint32_t k)
{
    uint32_t c = ctx().knobs.fc_topk_first_columns ? ctx().knobs.fc_topk_first_columns : 2048;
    c = std::max(c, (k + 127) / 128 * 128);   // at least k candidates for the first bound
    c = (c + 127) / 128 * 128;
    // when the first block would be most of the layer anyway, the whole layer goes through the scratch matrix
    return (n <= c + c / 2) ? n : c;
}

struct LayerWorkspace {
    float* block_scores;   // [batch][ld0]
    uint64_t* best;        // [batch][k]
    uint32_t* row_bound;   // [batch]   (row_bound, cand_count and row_flag are cleared together)
    uint32_t* cand_count;  // [batch]
    uint32_t* row_flag;    // [batch]
    uint32_t* overflow;    // [64] unused flag word of the shared epilogue
    uint64_t* cand;        // [batch][cap]
    size_t bytes;
};

static LayerWorkspace layer_layout(void* base, uint32_t batch, uint32_t n0, uint32_t k, uint32_t cap, bool ranges)
{
    LayerWorkspace w;
    char* p = (char*)base;
    const uint32_t ld0 = (n0 + 3) / 4 * 4;
    w.block_scores = (float*)p;
    p += align256((size_t)batch * ld0 * sizeof(float));
    w.best = (uint64_t*)p;
    p += align256((size_t)batch * k * sizeof(uint64_t));
    w.row_bound = (uint32_t*)p;
    w.cand_count = w.row_bound + batch;
    w.row_flag = w.cand_count + batch;
    w.overflow = w.row_flag + batch;
    p += align256(((size_t)3 * batch + 64) * sizeof(uint32_t));
    w.cand = (uint64_t*)p;
    if (ranges) p += align256((size_t)batch * cap * sizeof(uint64_t));
    w.bytes = (size_t)(p - (char*)base);
    return w;
}

static bool layer_activation_supported(uint32_t act, const dsx_act_params* params)
{
    switch (act) {
    case DSX_ACT_SIGMOID:
    case DSX_ACT_TANH:
    case DSX_ACT_RELU:
    case DSX_ACT_LINEAR: return true;
    case DSX_ACT_LRELU: return (params ? params->slope : 0.01f) > 0.0f;
    default: return false;
    }
}

}  // namespace dsx

using namespace dsx;

extern "C" {

int dsx_testing_set_fc_topk_first_columns(uint32_t columns)
{
    ctx().knobs.fc_topk_first_columns = std::min(columns, 131072u);   // the first block's filter bitmap lives in LDS
    return DSX_OK;
}

int dsx_testing_set_fc_topk_candidate_capacity(uint32_t words)
{
    DSX_CHECK_ARG(words == 0 || (words >= 64 && words <= kLayerCandCap), "dsx_testing_set_fc_topk_candidate_capacity: %u words (64..%u)", words, kLayerCandCap);
    ctx().knobs.fc_topk_candidate_capacity = words;
    return DSX_OK;
}

int dsx_fc_topk_flagged(int reset)
{
    if (!g_layer_flagged) return 0;
    int seen = 0;
    for (int i = 0; i < kFlagWords; i++) {
        seen |= *(volatile uint32_t*)&g_layer_flagged[i] != 0;
        if (reset) *(volatile uint32_t*)&g_layer_flagged[i] = 0;
    }
    return seen;
}

int dsx_fc_topk_flagged_for(const float* W, int reset)
{
    if (!g_layer_flagged) return 0;
    const int i = layer_flag_slot(W, false);
    if (i < 0) return 0;
    const int seen = *(volatile uint32_t*)&g_layer_flagged[i] != 0;
    if (reset) *(volatile uint32_t*)&g_layer_flagged[i] = 0;
    return seen;
}

int dsx_fc_topk_supported(uint32_t ldx, const float* X, uint32_t activation, const dsx_act_params* params, const float* filter_mul)
{
    return layer_activation_supported(activation, params) && filter_mul == nullptr && ((uintptr_t)X % 16) == 0 && (ldx % 4) == 0;
}

}  // extern "C"

// x_planes / w_planes (both or neither): the operands as dsx_fc_split leaves them; the products then come from the split-product
// kernel.  X and W are needed either way (rows whose lists fill up are recomputed from them, in fp32).
static int fc_topk_common(const float* X, uint32_t ldx, const float* W, const float* bias, uint32_t batch, uint32_t kdim, uint32_t n,
                          uint32_t activation, const dsx_act_params* params, uint32_t k, float* keys, uint32_t* values, uint32_t position,
                          const uint32_t* index, const uint64_t* filter_start, const uint64_t* filter_end, const uint32_t* filter_index,
                          const void* x_planes, const void* w_planes)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(X && W && keys && values, "dsx_fc_topk: null device pointer");
    DSX_CHECK_ARG(kdim > 0 && n > 0 && ldx >= kdim, "dsx_fc_topk: k = %u, n = %u, ldx = %u", kdim, n, ldx);
    DSX_CHECK_ARG(k >= 1 && k <= 256, "dsx_fc_topk: k = %u is outside 1..256", k);
    DSX_CHECK_ARG(!filter_index || (filter_start && filter_end), "dsx_fc_topk: filter_index without filter_start / filter_end");
    if (!dsx_fc_topk_supported(ldx, X, activation, params, nullptr))
        return set_error(DSX_EUNSUPPORTED, "dsx_fc_topk: activation %u is not monotone (sigmoid, tanh, ReLU, leaky ReLU with a positive slope, "
                         "linear are), or X is not 16-byte aligned with a pitch that is a multiple of 4: use dsx_fc_forward + dsx_topk_filtered",
                         activation);
    if (batch == 0) return DSX_OK;
    if (!g_layer_flagged) {
        DSX_HIP(hipHostMalloc((void**)&g_layer_flagged, kFlagWords * sizeof(uint32_t), hipHostMallocMapped));
        for (int i = 0; i < kFlagWords; i++) g_layer_flagged[i] = 0;
        at_shutdown(layer_flags_release);
    }
    uint32_t* const flag_word = g_layer_flagged + layer_flag_slot(W, true);
    const uint32_t cap = ctx().knobs.fc_topk_candidate_capacity ? ctx().knobs.fc_topk_candidate_capacity : kLayerCandCap;   // tests lower it to reach the overflow path with small inputs
    const uint32_t n0 = layer_first_columns(n, k);
    const bool ranges = n0 < n;
    const size_t need = layer_layout(nullptr, batch, n0, k, cap, ranges).bytes;
    LibScratch& ws = g_layer_ws_of[current_lane()];
    if (int rc = lib_scratch_reserve(ws, need, "dsx_fc_topk workspace")) return rc;
    const LayerWorkspace w = layer_layout(ws.ptr, batch, n0, k, cap, ranges);
    const uint32_t ld0 = (n0 + 3) / 4 * 4;
    hipStream_t s = ctx().stream;

    // first block: the layer as a matrix, then the scanning top-K (filtered: indexes beyond the block are ignored)
    const uint32_t wrows = split_rows_padded(n);
    int rc = x_planes ? fc_split_run(x_planes, w_planes, wrows, 0, bias, w.block_scores, ld0, batch, kdim, n0, 0, activation, params, nullptr, nullptr)
                      : fc_run(X, ldx, W, n, 0, bias, w.block_scores, ld0, batch, kdim, n0, 0, activation, params);
    if (rc) return rc;
    if (!ranges)
        return topk_run(w.block_scores, ld0, n0, batch, k, keys, values, position, index, filter_start, filter_end, filter_index, nullptr, 0,
                        nullptr, 0, 0, 0);
    const uint32_t clear_words = 3 * batch + 64;
    hipLaunchKernelGGL(layer_clear_kernel, dim3((clear_words + 255) / 256), dim3(256), 0, s, w.row_bound, clear_words);
    DSX_LAUNCH_CHECK("layer_clear_kernel");
    rc = topk_run(w.block_scores, ld0, n0, batch, k, nullptr, nullptr, position, index, filter_start, filter_end, filter_index, nullptr, 0,
                  w.best, 1, 0, 1, w.row_bound);
    if (rc) return rc;

    // A bound taken over `done` columns lets about k * width / done of the next `width` columns pass: ranges grow by a factor that
    // keeps that near an eighth of a list (the sample's own items, which score high and pass as well, come on top).
    const uint32_t growth = std::max(4u, cap / (8 * k));
    uint32_t done = n0;
    while (done < n) {
        uint32_t ncols = (uint32_t)std::min<uint64_t>((uint64_t)n - done, (uint64_t)done * growth / 128 * 128);
        if (n - done - ncols < 128) ncols = n - done;   // no sliver of a last range
        CandArgs cand{};
        cand.row_bound = w.row_bound;
        cand.cand = w.cand;
        cand.cand_count = w.cand_count;
        cand.cand_cap = cap;
        cand.col_offset = done;
        cand.overflow = w.overflow;
        cand.act = activation;
        cand.slope = params ? params->slope : 0.01f;
        cand.alpha = params ? params->alpha : 1.0f;
        cand.lambda = params ? params->lambda : 1.0f;
        rc = x_planes ? fc_split_candidates_run(x_planes, w_planes, wrows, done, batch, kdim, ncols, cand, true, bias ? bias + done : nullptr)
                      : fc_layer_candidates_run(X, ldx, W + done, n, bias ? bias + done : nullptr, batch, kdim, ncols, cand);
        if (rc) return rc;
        done += ncols;
        LayerRefresh r{};
        r.best = w.best; r.cand = w.cand; r.cand_count = w.cand_count; r.cap = cap; r.k = k;
        r.row_bound = w.row_bound; r.row_flag = w.row_flag; r.flagged_total = flag_word;
        r.position = position; r.index = index; r.fstart = filter_start; r.fend = filter_end; r.fidx = filter_index;
        if (done == n) {
            r.keys = keys;
            r.values = values;
        }
        r.X = X; r.W = W; r.bias = bias; r.ldx = ldx; r.ldw = n; r.kdim = kdim; r.n = n; r.first_columns = n0;
        r.act = activation; r.slope = cand.slope; r.alpha = cand.alpha; r.lambda = cand.lambda;
        rc = layer_refresh_run(r, batch);
        if (rc) return rc;
    }
    return DSX_OK;
}

extern "C" {

int dsx_fc_topk(const float* X, uint32_t ldx, const float* W, const float* bias, uint32_t batch, uint32_t kdim, uint32_t n,
                uint32_t activation, const dsx_act_params* params, uint32_t k, float* keys, uint32_t* values, uint32_t position,
                const uint32_t* index, const uint64_t* filter_start, const uint64_t* filter_end, const uint32_t* filter_index)
{
    return fc_topk_common(X, ldx, W, bias, batch, kdim, n, activation, params, k, keys, values, position, index, filter_start, filter_end,
                          filter_index, nullptr, nullptr);
}

int dsx_fc_topk_split(const float* X, uint32_t ldx, const float* W, const void* x_planes, const void* w_planes, const float* bias,
                      uint32_t batch, uint32_t kdim, uint32_t n, uint32_t activation, const dsx_act_params* params, uint32_t k, float* keys,
                      uint32_t* values, uint32_t position, const uint32_t* index, const uint64_t* filter_start, const uint64_t* filter_end,
                      const uint32_t* filter_index)
{
    DSX_CHECK_ARG(x_planes && w_planes, "dsx_fc_topk_split: null planes");
    DSX_CHECK_ARG(((uintptr_t)x_planes % 16) == 0 && ((uintptr_t)w_planes % 16) == 0, "dsx_fc_topk_split: planes must be 16-byte aligned");
    return fc_topk_common(X, ldx, W, bias, batch, kdim, n, activation, params, k, keys, values, position, index, filter_start, filter_end,
                          filter_index, x_planes, w_planes);
}

}  // extern "C"
