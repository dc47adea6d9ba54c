// dsx_topk.hip — per-row top-K of a score matrix, plain, KNN-padded, key/value and filtered.
//
// Design (wave64, one 256-lane workgroup per (row, column segment)):
//   * every (score, column) pair is packed into one 64-bit unsigned word, order-preserving for the score in the high half
//     and the complemented column in the low half, so "largest word" == "highest score, then lowest column": the whole
//     selection runs on unsigned 64-bit max/min and the result order is total and reproducible;
//   * each wavefront streams 128-bit loads of its share of the row and keeps a running top-L list (L = 64, 128 or 256
//     >= k) in registers, one to four words per lane, sorted descending across (register, lane);
//   * a score enters only if it beats the list's current k-th word; survivors are compacted with a 64-bit ballot into a
//     per-wave LDS staging area and, once L of them are waiting, bitonic-sorted (cross-lane exchanges) and merged into the
//     register list, which tightens the threshold;
//   * the filter (items to multiply, normally by 0, e.g. the sample's own inputs) is a per-segment bitmap in LDS:
//     listed columns are dropped from the scan and re-injected once with score * multiplier;
//   * the four wave lists are merged through LDS; rows split over several segments write packed partial lists that a
//     second small kernel merges.
#include <algorithm>
#include "dsx_device.h"
#include "dsx_internal.h"

namespace dsx {

constexpr int kTopkThreads = 256;
constexpr int kTopkWaves = kTopkThreads / kWave;
constexpr uint32_t kMaxBitmapBits = 256 * 1024;   // 32 KiB of LDS per workgroup

__device__ __forceinline__ uint64_t pack_score(float key, uint32_t col)
{
    key += 0.0f;   // -0.0 -> +0.0 so that both zeros tie and fall back to the column order
    uint32_t u = __float_as_uint(key);
    u ^= (uint32_t)((int32_t)u >> 31) | 0x80000000u;
    return ((uint64_t)u << 32) | (uint32_t)~col;
}

__device__ __forceinline__ void unpack_score(uint64_t p, float& key, uint32_t& col)
{
    uint32_t u = (uint32_t)(p >> 32);
    u ^= ((u >> 31) - 1u) | 0x80000000u;
    key = __uint_as_float(u);
    col = ~(uint32_t)p;
}

__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int mask)
{
    uint32_t lo = (uint32_t)__shfl_xor((int)(uint32_t)v, mask, kWave);
    uint32_t hi = (uint32_t)__shfl_xor((int)(uint32_t)(v >> 32), mask, kWave);
    return ((uint64_t)hi << 32) | lo;
}

__device__ __forceinline__ uint64_t shfl_u64(uint64_t v, int src)
{
    uint32_t lo = (uint32_t)__shfl((int)(uint32_t)v, src, kWave);
    uint32_t hi = (uint32_t)__shfl((int)(uint32_t)(v >> 32), src, kWave);
    return ((uint64_t)hi << 32) | lo;
}

__device__ __forceinline__ uint64_t umax64(uint64_t a, uint64_t b) { return a > b ? a : b; }
__device__ __forceinline__ uint64_t umin64(uint64_t a, uint64_t b) { return a > b ? b : a; }

// One compare-exchange layer of a bitonic network over 64*R words held as v[r] in lane `lane` (position r*64 + lane).
// J: partner distance, K: size of the monotone blocks being built, DESC: direction of the final order.
template <int R, bool DESC, int K, int J>
__device__ __forceinline__ void bitonic_layer(uint64_t (&v)[R], uint32_t lane)
{
    if constexpr (J >= kWave) {
        constexpr int JR = J / kWave;
#pragma unroll
        for (int r = 0; r < R; r++) {
            if ((r & JR) == 0) {
                const int r2 = r | JR;
                const bool desc_block = (((r * kWave) & K) == 0) == DESC;
                const uint64_t a = v[r], b = v[r2];
                const uint64_t mx = umax64(a, b), mn = umin64(a, b);
                v[r] = desc_block ? mx : mn;
                v[r2] = desc_block ? mn : mx;
            }
        }
    } else {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint32_t p = r * kWave + lane;
            const bool desc_block = ((p & K) == 0) == DESC;
            const bool lower = (lane & J) == 0;
            const uint64_t other = shfl_xor_u64(v[r], J);
            v[r] = (lower == desc_block) ? umax64(v[r], other) : umin64(v[r], other);
        }
    }
}

template <int R, bool DESC, int K, int J> struct BitonicJ {
    static __device__ __forceinline__ void run(uint64_t (&v)[R], uint32_t lane)
    {
        bitonic_layer<R, DESC, K, J>(v, lane);
        if constexpr (J > 1) BitonicJ<R, DESC, K, J / 2>::run(v, lane);
    }
};

template <int R, bool DESC, int K> struct BitonicK {
    static __device__ __forceinline__ void run(uint64_t (&v)[R], uint32_t lane)
    {
        if constexpr (K > 2) BitonicK<R, DESC, K / 2>::run(v, lane);
        BitonicJ<R, DESC, K, K / 2>::run(v, lane);
    }
};

// Full sort of 64*R words.
template <int R, bool DESC> __device__ __forceinline__ void bitonic_sort(uint64_t (&v)[R], uint32_t lane)
{
    BitonicK<R, DESC, kWave * R>::run(v, lane);
}

// Sorts a bitonic sequence of 64*R words descending.
template <int R> __device__ __forceinline__ void bitonic_merge_desc(uint64_t (&v)[R], uint32_t lane)
{
    BitonicJ<R, true, kWave * R, kWave * R / 2>::run(v, lane);
}

// Running top-L list of one wavefront plus its LDS staging area.
template <int R> struct WaveTopK {
    static constexpr int L = kWave * R;
    static constexpr int kStageWords = L + kWave;

    uint64_t q[R];        // sorted descending over position r*64 + lane; 0 = empty slot
    uint64_t thr;         // current k-th word: candidates must be strictly larger
    float thr_key;        // its score: cheap first test is score >= thr_key
    uint32_t count;       // staged candidates (wave-uniform)
    uint64_t* stage;      // LDS, kStageWords words, private to this wave
    uint32_t lane;
    uint32_t k;

    __device__ __forceinline__ void init(uint64_t* stage_, uint32_t lane_, uint32_t k_)
    {
#pragma unroll
        for (int r = 0; r < R; r++) q[r] = 0;
        thr = 0;
        thr_key = -__builtin_inff();
        count = 0;
        stage = stage_;
        lane = lane_;
        k = k_;
    }

    // Merge the first min(count, L) staged words into the list.
    __device__ __forceinline__ void flush()
    {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        uint64_t c[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint32_t p = r * kWave + lane;
            c[r] = (p < count) ? stage[p] : 0;
        }
        bitonic_sort<R, false>(c, lane);                       // ascending
#pragma unroll
        for (int r = 0; r < R; r++) q[r] = umax64(q[r], c[r]);   // top L of the union, bitonic
        bitonic_merge_desc<R>(q, lane);
        // k-th word -> threshold
        const uint32_t kr = (k - 1) / kWave, kl = (k - 1) % kWave;
        uint64_t t = q[0];
#pragma unroll
        for (int r = 1; r < R; r++) t = (kr == (uint32_t)r) ? q[r] : t;
        thr = shfl_u64(t, (int)kl);
        if (thr != 0) {
            float key;
            uint32_t col;
            unpack_score(thr, key, col);
            thr_key = key;
        }
        // keep what did not fit
        const uint32_t rest = (count > (uint32_t)L) ? count - L : 0;
        uint64_t keep = 0;
        if (lane < rest) keep = stage[L + lane];
        __builtin_amdgcn_wave_barrier();
        if (lane < rest) stage[lane] = keep;
        count = rest;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }

    // Offer one word per lane (valid lanes only).  All 64 lanes must call this together.
    __device__ __forceinline__ void offer(bool valid, uint64_t word)
    {
        const bool cand = valid && (word > thr);
        const uint64_t m = __ballot(cand);
        if (m == 0) return;
        const uint64_t below = m & ((1ull << lane) - 1ull);
        if (cand) stage[count + __popcll(below)] = word;
        count += (uint32_t)__popcll(m);
        if (count >= (uint32_t)L) flush();
    }

    __device__ __forceinline__ void finish()
    {
        while (count > 0) flush();
    }
};

struct TopKArgs {
    const float* in;        // [batch][pitch]
    uint32_t pitch;         // elements between rows
    uint32_t width;         // candidate columns per row (<= pitch)
    uint32_t k;
    uint32_t segments;      // workgroups per row
    uint32_t col_offset;    // added to the reported column (column blocks of a larger matrix)
    // filter (all NULL when unfiltered)
    uint32_t position;
    const uint32_t* index;
    const uint64_t* fstart;
    const uint64_t* fend;
    const uint32_t* fidx;
    const float* fmul;
    // results: either final (keys/values, pitch k) or packed partial lists
    float* keys;
    uint32_t* values;
    uint64_t* partial;          // [batch][partial_slots][k]
    uint32_t partial_slots;
    uint32_t partial_slot0;     // this launch writes slots partial_slot0 + segment
};

template <int R>
__device__ __forceinline__ void write_final(const uint64_t (&q)[R], uint32_t lane, uint32_t k, uint32_t col_offset, float* keys,
                                            uint32_t* values)
{
#pragma unroll
    for (int r = 0; r < R; r++) {
        const uint32_t p = r * kWave + lane;
        if (p < k) {
            float key = -kMaxValue;   // engine/kernels.cu:3221-3224: unfilled slots
            uint32_t col = 0;
            if (q[r] != 0) {
                unpack_score(q[r], key, col);
                col += col_offset;
            }
            keys[p] = key;
            values[p] = col;
        }
    }
}

template <int R, bool FILTERED>
__global__ __launch_bounds__(kTopkThreads) void topk_scan_kernel(TopKArgs a)
{
    using List = WaveTopK<R>;
    __shared__ uint64_t sStage[kTopkWaves][List::kStageWords];
    extern __shared__ uint32_t sBitmap[];

    const uint32_t b = blockIdx.x;
    const uint32_t seg = blockIdx.y;
    const uint32_t wave = threadIdx.x / kWave;
    const uint32_t lane = threadIdx.x % kWave;
    const float* row = a.in + (uint64_t)b * a.pitch;

    // Split the row into an unaligned head (< 4 columns), a body of 16-byte groups and a tail (< 4 columns).
    const uint32_t mis = (uint32_t)(((uintptr_t)row >> 2) & 3);
    uint32_t head = (4 - mis) & 3;
    if (head > a.width) head = a.width;
    const uint32_t nvec = (a.width - head) / 4;
    const uint32_t tail0 = head + nvec * 4;
    const uint32_t gps = (nvec + a.segments - 1) / a.segments;      // groups per segment
    const uint32_t g0 = min(seg * gps, nvec), g1 = min(g0 + gps, nvec);
    const uint32_t lo = (seg == 0) ? 0 : head + 4 * g0;
    const uint32_t hi = (seg == a.segments - 1) ? a.width : head + 4 * g1;

    List list;
    list.init(sStage[wave], lane, a.k);

    // Software pipeline: the first four 16-byte groups of this lane are requested before the filter is built (its chain of
    // dependent loads would otherwise sit in front of the scan), and inside the loop the next four are requested before the
    // current four are examined.
    const float4* body = reinterpret_cast<const float4*>(row + head);
    const uint32_t step = kTopkThreads;
    uint32_t span = g0;   // block-uniform
    bool have = span + 4 * step <= g1;
    float4 cur0, cur1, cur2, cur3;
    cur0 = cur1 = cur2 = cur3 = make_float4(0.f, 0.f, 0.f, 0.f);
    if (have) {
        const uint32_t g = span + threadIdx.x;
        cur0 = body[g];
        cur1 = body[g + step];
        cur2 = body[g + 2 * step];
        cur3 = body[g + 3 * step];
    }

    if constexpr (FILTERED) {
        const uint32_t words = (hi - lo + 31) / 32;
        for (uint32_t i = threadIdx.x; i < words; i += kTopkThreads) sBitmap[i] = 0;
        __syncthreads();
        uint32_t r = a.position + b;
        if (a.index) r = a.index[r];
        const uint64_t fs = a.fstart[r], fe = a.fend[r];
        // Mark the listed columns; the lane that sets a bit first owns the entry and injects score * multiplier.
        for (uint64_t base = fs; base < fe; base += kTopkThreads) {
            const uint64_t t = base + threadIdx.x;
            bool own = false;
            uint64_t word = 0;
            if (t < fe) {
                const uint32_t col = a.fidx[t];
                if (col >= lo && col < hi) {
                    const uint32_t bit = 1u << ((col - lo) & 31);
                    const uint32_t old = atomicOr(&sBitmap[(col - lo) >> 5], bit);
                    if (!(old & bit)) {
                        const float mul = a.fmul ? a.fmul[t] : 0.0f;
                        const float v = mul * row[col];           // utils/Filters.cpp:62
                        own = !(v != v);                          // NaN never enters (it fails every comparison)
                        word = pack_score(v, col);
                    }
                }
            }
            list.offer(own, word);
        }
        __syncthreads();
    }

    auto filtered_out = [&](uint32_t col) -> bool {
        if constexpr (FILTERED) {
            return (sBitmap[(col - lo) >> 5] >> ((col - lo) & 31)) & 1u;
        } else {
            return false;
        }
    };

    auto consider4 = [&](const float4& v, uint32_t col) {
        const float t = list.thr_key;
        const bool any = (v.x >= t) | (v.y >= t) | (v.z >= t) | (v.w >= t);
        if (__ballot(any) == 0) return;
        const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int c = 0; c < 4; c++) {
            bool ok = e[c] >= list.thr_key;
            if (ok) ok = !filtered_out(col + c);
            list.offer(ok, pack_score(e[c], col + c));
        }
    };

    // Body: the block walks the segment in 4 KiB spans, wave w takes the w-th KiB of each span.
    while (have) {
        const uint32_t g = span + threadIdx.x;
        const uint32_t nspan = span + 4 * step;
        const bool have_next = nspan + 4 * step <= g1;
        float4 n0, n1, n2, n3;
        n0 = n1 = n2 = n3 = make_float4(0.f, 0.f, 0.f, 0.f);
        if (have_next) {
            const uint32_t gn = nspan + threadIdx.x;
            n0 = body[gn];
            n1 = body[gn + step];
            n2 = body[gn + 2 * step];
            n3 = body[gn + 3 * step];
        }
        consider4(cur0, head + 4 * g);
        consider4(cur1, head + 4 * (g + step));
        consider4(cur2, head + 4 * (g + 2 * step));
        consider4(cur3, head + 4 * (g + 3 * step));
        cur0 = n0;
        cur1 = n1;
        cur2 = n2;
        cur3 = n3;
        span = nspan;
        have = have_next;
    }
    for (; span < g1; span += step) {
        const uint32_t g = span + threadIdx.x;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        const bool in = g < g1;
        if (in) v = body[g];
        const float t = list.thr_key;
        const bool any = in && ((v.x >= t) | (v.y >= t) | (v.z >= t) | (v.w >= t));
        if (__ballot(any) == 0) continue;
        const float e[4] = {v.x, v.y, v.z, v.w};
        const uint32_t col = head + 4 * g;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            bool ok = in && (e[c] >= list.thr_key);
            if (ok) ok = !filtered_out(col + c);
            list.offer(ok, pack_score(e[c], col + c));
        }
    }
    // Head (segment 0) and tail (last segment): at most 3 + 3 columns, taken by wave 0.
    if (wave == 0) {
        uint32_t col = 0xffffffffu;
        if (seg == 0 && lane < head) col = lane;
        if (seg == a.segments - 1 && lane >= 32 && (lane - 32) < a.width - tail0) col = tail0 + (lane - 32);
        bool ok = col != 0xffffffffu;
        float v = 0.0f;
        if (ok) {
            v = row[col];
            ok = (v >= list.thr_key) && !filtered_out(col);
        }
        list.offer(ok, pack_score(v, col));
    }
    list.finish();

    // Merge the four wave lists: waves 1..3 publish their first k words, wave 0 takes them as candidates.
    __syncthreads();
    // staging areas are idle now; wave w > 0 publishes into its own area
    if (wave != 0) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint32_t p = r * kWave + lane;
            if (p < a.k) sStage[wave][p] = list.q[r];
        }
    }
    __syncthreads();
    if (wave != 0) return;
    for (uint32_t w = 1; w < kTopkWaves; w++) {
        for (uint32_t p0 = 0; p0 < a.k; p0 += kWave) {
            const uint32_t p = p0 + lane;
            uint64_t word = 0;
            if (p < a.k) word = sStage[w][p];
            // sStage[0] is wave 0's own staging area, distinct from the published lists of waves 1..3
            list.offer(word != 0, word);
        }
    }
    list.finish();

    if (a.partial) {
        uint64_t* dst = a.partial + ((uint64_t)b * a.partial_slots + a.partial_slot0 + seg) * a.k;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint32_t p = r * kWave + lane;
            if (p < a.k) {
                uint64_t word = list.q[r];
                if (word != 0 && a.col_offset != 0) {
                    float key;
                    uint32_t col;
                    unpack_score(word, key, col);
                    word = (word & 0xffffffff00000000ull) | (uint32_t)~(col + a.col_offset);
                }
                dst[p] = word;
            }
        }
    } else {
        write_final<R>(list.q, lane, a.k, a.col_offset, a.keys + (uint64_t)b * a.k, a.values + (uint64_t)b * a.k);
    }
}

// Second stage: one wavefront per row merges `slots` packed partial lists of k words each.
template <int R>
__global__ __launch_bounds__(kWave) void topk_merge_kernel(const uint64_t* partial, uint32_t slots, uint32_t k, float* keys,
                                                           uint32_t* values)
{
    using List = WaveTopK<R>;
    __shared__ uint64_t sStage[List::kStageWords];
    const uint32_t b = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    List list;
    list.init(sStage, lane, k);
    const uint64_t* src = partial + (uint64_t)b * slots * k;
    const uint32_t total = slots * k;
    for (uint32_t p0 = 0; p0 < total; p0 += kWave) {
        const uint32_t p = p0 + lane;
        uint64_t word = 0;
        if (p < total) word = src[p];
        list.offer(word != 0, word);
    }
    list.finish();
    write_final<R>(list.q, lane, k, 0, keys + (uint64_t)b * k, values + (uint64_t)b * k);
}

// In-place payload gather for the key/value overloads: values[b][j] holds a column number on entry.
template <typename V>
__global__ __launch_bounds__(256) void topk_gather_kernel(const V* in_values, V* values, uint32_t batch, uint32_t width, uint32_t k)
{
    const uint64_t pos = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (pos >= (uint64_t)batch * k) return;
    const uint32_t b = (uint32_t)(pos / k), j = (uint32_t)(pos % k);
    const uint32_t col = reinterpret_cast<const uint32_t*>(values)[pos];
    values[pos] = (j < width) ? in_values[(uint64_t)b * width + col] : (V)0;
}

static uint64_t* g_partial = nullptr;
static size_t g_partial_bytes = 0;

static int ensure_partial(size_t bytes)
{
    if (bytes <= g_partial_bytes) return DSX_OK;
    if (g_partial) {
        DSX_HIP(hipStreamSynchronize(ctx().stream));
        DSX_HIP(hipFree(g_partial));
        g_partial = nullptr;
        g_partial_bytes = 0;
    }
    hipError_t e = hipMalloc((void**)&g_partial, bytes);
    if (e != hipSuccess) return set_error(DSX_ENOMEM, "top-K: cannot allocate %zu bytes for partial lists: %s", bytes, hipGetErrorString(e));
    g_partial_bytes = bytes;
    return DSX_OK;
}

template <int R> static int launch_scan(const TopKArgs& a, uint32_t batch, bool filtered, size_t bitmap_bytes)
{
    dim3 grid(batch, a.segments);
    if (filtered)
        hipLaunchKernelGGL((topk_scan_kernel<R, true>), grid, dim3(kTopkThreads), bitmap_bytes, ctx().stream, a);
    else
        hipLaunchKernelGGL((topk_scan_kernel<R, false>), grid, dim3(kTopkThreads), 0, ctx().stream, a);
    DSX_LAUNCH_CHECK("topk_scan_kernel");
    return DSX_OK;
}

template <int R> static int launch_merge(const uint64_t* partial, uint32_t slots, uint32_t k, float* keys, uint32_t* values, uint32_t batch)
{
    hipLaunchKernelGGL((topk_merge_kernel<R>), dim3(batch), dim3(kWave), 0, ctx().stream, partial, slots, k, keys, values);
    DSX_LAUNCH_CHECK("topk_merge_kernel");
    return DSX_OK;
}

// Number of workgroups per row: enough to fill the device, and small enough segments for the LDS bitmap.
static uint32_t choose_segments(uint32_t batch, uint32_t width, bool filtered)
{
    uint32_t s = 1;
    const uint32_t target_blocks = (uint32_t)ctx().num_cus * 4;
    if (batch < target_blocks) s = (target_blocks + batch - 1) / batch;
    const uint32_t max_by_size = std::max(1u, width / 8192);   // keep at least 8192 columns per segment
    s = std::min(s, max_by_size);
    if (filtered) {
        const uint32_t need = (width + (kMaxBitmapBits - 64) - 1) / (kMaxBitmapBits - 64);
        s = std::max(s, need);
    }
    return std::max(1u, s);
}

int topk_merge(const uint64_t* partial, uint32_t slots, uint32_t k, float* keys, uint32_t* values, uint32_t batch);

int topk_run(const float* in, uint32_t pitch, uint32_t width, uint32_t batch, uint32_t k, float* keys, uint32_t* values,
             uint32_t position, const uint32_t* index, const uint64_t* fstart, const uint64_t* fend, const uint32_t* fidx,
             const float* fmul, uint32_t col_offset, uint64_t* partial, uint32_t partial_slots, uint32_t partial_slot0,
             uint32_t forced_segments)
{
    const bool filtered = fidx != nullptr;
    TopKArgs a{};
    a.in = in;
    a.pitch = pitch;
    a.width = width;
    a.k = k;
    a.col_offset = col_offset;
    a.position = position;
    a.index = index;
    a.fstart = fstart;
    a.fend = fend;
    a.fidx = fidx;
    a.fmul = fmul;
    a.keys = keys;
    a.values = values;
    a.segments = forced_segments ? forced_segments : choose_segments(batch, width, filtered);
    const uint32_t nvec_max = width / 4 + 1;
    const uint32_t gps = (nvec_max + a.segments - 1) / a.segments;
    const size_t bitmap_bytes = filtered ? ((size_t)(4 * gps + 8 + 31) / 32) * 4 + 16 : 0;
    if (partial) {
        a.partial = partial;
        a.partial_slots = partial_slots;
        a.partial_slot0 = partial_slot0;
    } else if (a.segments > 1) {
        int rc = ensure_partial((size_t)batch * a.segments * k * sizeof(uint64_t));
        if (rc) return rc;
        a.partial = g_partial;
        a.partial_slots = a.segments;
        a.partial_slot0 = 0;
    }
    int rc;
    if (k <= 64)
        rc = launch_scan<1>(a, batch, filtered, bitmap_bytes);
    else if (k <= 128)
        rc = launch_scan<2>(a, batch, filtered, bitmap_bytes);
    else
        rc = launch_scan<4>(a, batch, filtered, bitmap_bytes);
    if (rc) return rc;
    if (!partial && a.segments > 1) return topk_merge(a.partial, a.segments, k, keys, values, batch);
    return DSX_OK;
}

int topk_merge(const uint64_t* partial, uint32_t slots, uint32_t k, float* keys, uint32_t* values, uint32_t batch)
{
    if (k <= 64) return launch_merge<1>(partial, slots, k, keys, values, batch);
    if (k <= 128) return launch_merge<2>(partial, slots, k, keys, values, batch);
    return launch_merge<4>(partial, slots, k, keys, values, batch);
}

static int check_topk(const char* fn, const float* in, const float* keys, const void* values, uint32_t width, uint32_t k)
{
    DSX_CHECK_ARG(in && keys && values, "%s: null device pointer", fn);
    DSX_CHECK_ARG(k >= 1 && k <= 256, "%s: k = %u is outside 1..256", fn, k);
    DSX_CHECK_ARG(width >= 1, "%s: width is 0", fn);
    return DSX_OK;
}

}  // namespace dsx

using namespace dsx;

extern "C" {

int dsx_topk(const float* in, float* keys, uint32_t* values, uint32_t batch, uint32_t width, uint32_t k)
{
    DSX_REQUIRE_INIT();
    int rc = check_topk("dsx_topk", in, keys, values, width, k);
    if (rc) return rc;
    if (batch == 0) return DSX_OK;
    return topk_run(in, width, width, batch, k, keys, values, 0, nullptr, nullptr, nullptr, nullptr, nullptr, 0, nullptr, 0, 0, 0);
}

int dsx_knn_topk(const float* in, float* keys, uint32_t* values, uint32_t batch, uint32_t width, uint32_t width_padding, uint32_t k)
{
    DSX_REQUIRE_INIT();
    int rc = check_topk("dsx_knn_topk", in, keys, values, width, k);
    if (rc) return rc;
    DSX_CHECK_ARG(width_padding < width, "dsx_knn_topk: padding %u leaves no column of %u", width_padding, width);
    if (batch == 0) return DSX_OK;
    return topk_run(in, width, width - width_padding, batch, k, keys, values, 0, nullptr, nullptr, nullptr, nullptr, nullptr, 0, nullptr,
                    0, 0, 0);
}

int dsx_topk_filtered(const float* in, float* keys, uint32_t* values, uint32_t batch, uint32_t width, uint32_t k, uint32_t position,
                      const uint32_t* index, const uint64_t* filter_start, const uint64_t* filter_end, const uint32_t* filter_index,
                      const float* filter_mul)
{
    DSX_REQUIRE_INIT();
    int rc = check_topk("dsx_topk_filtered", in, keys, values, width, k);
    if (rc) return rc;
    DSX_CHECK_ARG(filter_start && filter_end && filter_index, "dsx_topk_filtered: null filter arrays (use dsx_topk for an unfiltered call)");
    if (batch == 0) return DSX_OK;
    return topk_run(in, width, width, batch, k, keys, values, position, index, filter_start, filter_end, filter_index, filter_mul, 0,
                    nullptr, 0, 0, 0);
}

int dsx_topk_kv_f32(const float* in_keys, const float* in_values, float* keys, float* values, uint32_t batch, uint32_t width, uint32_t k)
{
    DSX_REQUIRE_INIT();
    int rc = check_topk("dsx_topk_kv_f32", in_keys, keys, values, width, k);
    if (rc) return rc;
    DSX_CHECK_ARG(in_values, "dsx_topk_kv_f32: null input values");
    if (batch == 0) return DSX_OK;
    rc = topk_run(in_keys, width, width, batch, k, keys, reinterpret_cast<uint32_t*>(values), 0, nullptr, nullptr, nullptr, nullptr,
                  nullptr, 0, nullptr, 0, 0, 0);
    if (rc) return rc;
    const uint64_t n = (uint64_t)batch * k;
    hipLaunchKernelGGL(topk_gather_kernel<float>, dim3((uint32_t)((n + 255) / 256)), dim3(256), 0, ctx().stream, in_values, values, batch,
                       width, k);
    DSX_LAUNCH_CHECK("topk_gather_kernel");
    return DSX_OK;
}

int dsx_topk_kv_u32(const float* in_keys, const uint32_t* in_values, float* keys, uint32_t* values, uint32_t batch, uint32_t width,
                    uint32_t k)
{
    DSX_REQUIRE_INIT();
    int rc = check_topk("dsx_topk_kv_u32", in_keys, keys, values, width, k);
    if (rc) return rc;
    DSX_CHECK_ARG(in_values, "dsx_topk_kv_u32: null input values");
    if (batch == 0) return DSX_OK;
    rc = topk_run(in_keys, width, width, batch, k, keys, values, 0, nullptr, nullptr, nullptr, nullptr, nullptr, 0, nullptr, 0, 0, 0);
    if (rc) return rc;
    const uint64_t n = (uint64_t)batch * k;
    hipLaunchKernelGGL(topk_gather_kernel<uint32_t>, dim3((uint32_t)((n + 255) / 256)), dim3(256), 0, ctx().stream, in_values, values,
                       batch, width, k);
    DSX_LAUNCH_CHECK("topk_gather_kernel");
    return DSX_OK;
}

}  // extern "C"
