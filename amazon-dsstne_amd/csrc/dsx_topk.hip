// dsx_topk.hip — per-row top-K of a score matrix, plain, KNN-padded, key/value and filtered.
//
// Design (wave64, one 256-lane workgroup per (row, column segment)):
//   * every (score, column) pair is packed into one 64-bit unsigned word, order-preserving for the score in the high half
//     and the complemented column in the low half, so "largest word" == "highest score, then lowest column": the whole
//     selection runs on unsigned 64-bit max/min and the result order is total and reproducible;
//   * each wavefront streams 128-bit loads of its share of the row, two spans of eight loads per lane in flight, and keeps
//     a running top-L list (L = 64, 128 or 256 >= k) in registers, one to four words per lane, sorted descending across
//     (register, lane);
//   * a score enters only if it beats the list's current k-th word; the common case costs three vector instructions per
//     16-byte group; survivors are compacted with a 64-bit ballot into a per-wave LDS staging area and, once L of them are
//     waiting, bitonic-sorted (cross-lane exchanges) and merged into the register list, which tightens the threshold;
//   * for k <= 128 the threshold is primed before the scan from the k-th best of the lanes' first-span maxima (a binary
//     search over key bits), so a 27k-column row stages about forty words, no wave ever sorts, and the final order comes
//     from counting, for each staged word, how many staged words are larger;
//   * the kernel is bound by instruction issue as much as by HBM (four waves per SIMD run the same phases in step), so the
//     code keeps rarely-taken work (packing, filter lookups) inside wave-uniform branches;
//   * the filter (items to multiply, normally by 0, e.g. the sample's own inputs) is a per-segment bitmap in LDS:
//     listed columns are dropped from the scan and injected once, after the scan, with score * multiplier;
//   * rows split over several segments write packed partial lists that a second small kernel merges.
#include <algorithm>
#include <type_traits>
#include "dsx_device.h"
#include "dsx_internal.h"

namespace dsx {

constexpr int kTopkThreads = 256;
constexpr int kTopkWaves = kTopkThreads / kWave;
constexpr uint32_t kMaxBitmapBits = 256 * 1024;   // 32 KiB of LDS per workgroup

__device__ __forceinline__ uint64_t pack_score(float key, uint32_t col)
{
    return ((uint64_t)score_key(key) << 32) | (uint32_t)~col;
}

// A lower bound of the k-th largest of the wave's 64*N keys, exact in its upper 20 bits (0 if k > 64*N): at least k keys are
// >= the result.  A radix-4 search over key bits 31..12; each step is three vector compares per key and scalar bookkeeping.
// Twelve bits of slack admit a handful of extra candidates, and save a third of a dependent chain that every wave runs
// before it can ask for more data.
template <int N> __device__ __forceinline__ uint32_t wave_kth_key(const uint32_t (&key)[N], uint32_t k)
{
    uint32_t t = 0;
#pragma unroll 1
    for (int bit = 30; bit >= 12; bit -= 2) {
        const uint32_t c1 = t | (1u << bit), c2 = t | (2u << bit), c3 = t | (3u << bit);
        uint32_t n1 = 0, n2 = 0, n3 = 0;
#pragma unroll
        for (int n = 0; n < N; n++) {
            n1 += (uint32_t)__popcll(__ballot(key[n] >= c1));
            n2 += (uint32_t)__popcll(__ballot(key[n] >= c2));
            n3 += (uint32_t)__popcll(__ballot(key[n] >= c3));
        }
        t = (n3 >= k) ? c3 : (n2 >= k) ? c2 : (n1 >= k) ? c1 : t;
    }
    return t;
}

__device__ __forceinline__ void unpack_score(uint64_t p, float& key, uint32_t& col)
{
    key = key_score((uint32_t)(p >> 32));
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
    static constexpr int kBurst = 5 * kWave;            // most words staged between two checks of the fill level
    static constexpr int kStageWords = L + kBurst;

    uint64_t q[R];        // sorted descending over position r*64 + lane; 0 = empty slot
    uint64_t thr;         // current k-th word: candidates must be strictly larger
    float thr_key;        // its score: cheap first test is score >= thr_key
    float thr_above;      // the next score above thr_key
    uint32_t thr_col;     // the k-th word's column (0xffffffff while the threshold is a bare score bound)
    uint32_t count;       // staged candidates (wave-uniform)
    bool flushed;         // the register list holds something
    uint64_t* stage;      // LDS, kStageWords words, private to this wave
    uint32_t lane;
    uint32_t k;

    __device__ __forceinline__ void init(uint64_t* stage_, uint32_t lane_, uint32_t k_)
    {
#pragma unroll
        for (int r = 0; r < R; r++) q[r] = 0;
        thr = 0;
        thr_key = -__builtin_inff();
        thr_above = -__builtin_inff();
        thr_col = 0xffffffffu;
        count = 0;
        flushed = false;
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
        flushed = true;
        const uint32_t kr = (k - 1) / kWave, kl = (k - 1) % kWave;
        uint64_t t = q[0];
#pragma unroll
        for (int r = 1; r < R; r++) t = (kr == (uint32_t)r) ? q[r] : t;
        raise_threshold(shfl_u64(t, (int)kl));
        // keep what did not fit: move it to the front, 64 words at a time (source and destination of one step never overlap
        // because L >= 64, and later sources lie above every earlier destination)
        const uint32_t rest = (count > (uint32_t)L) ? count - L : 0;
        for (uint32_t i = 0; i < rest; i += kWave) {
            uint64_t keep = 0;
            if (i + lane < rest) keep = stage[L + i + lane];
            __builtin_amdgcn_wave_barrier();
            if (i + lane < rest) stage[i + lane] = keep;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
        count = rest;
    }

    // Words at or below t can no longer reach the top k.
    __device__ __forceinline__ void raise_threshold(uint64_t t)
    {
        if (t > thr) {
            thr = t;
            float key;
            uint32_t col;
            unpack_score(t, key, col);
            thr_key = key;
            thr_above = key_score((uint32_t)(t >> 32) + 1u);   // above +inf this is NaN, which nothing reaches
            thr_col = col;
        }
    }

    // Lowest score a column at or beyond first_col needs.  A score equal to the k-th one wins only with a smaller column, so once
    // the k-th word's column lies before first_col, ties are out: in a row of saturated scores (thousands of columns at exactly
    // 1.0) the scan then skips every group with one compare, like any other row.
    __device__ __forceinline__ float admission_score(uint32_t first_col) const
    {
        return (thr_col < first_col) ? thr_above : thr_key;
    }

    // Every word whose score key is below t can no longer reach the top k (t must be the key of a real score).
    __device__ __forceinline__ void prime(uint32_t t)
    {
        const uint64_t w = ((uint64_t)t << 32) - 1;
        if (w > thr) {
            thr = w;
            thr_key = key_score(t);
            thr_col = 0xffffffffu;
        }
    }

    // The same with a column: at least k real words are >= w (w need not be a real word itself).  Scores equal to w's then only
    // pass with a column at or before w's, which admission_score turns into "strictly above" for everything that lies behind it.
    __device__ __forceinline__ void prime_word(uint64_t w)
    {
        if (w - 1 > thr) {
            thr = w - 1;
            float key;
            uint32_t col;
            unpack_score(w, key, col);
            thr_key = key;
            thr_above = key_score((uint32_t)(w >> 32) + 1u);
            thr_col = col;
        }
    }

    // Stage the lanes' words that beat the threshold.  All 64 lanes must call this together.  Nothing is merged here: after
    // at most five calls the caller runs drain(), which keeps count < L between bursts.
    __device__ __forceinline__ void stage_only(bool valid, uint64_t word)
    {
        const bool cand = valid && (word > thr);
        const uint64_t m = __ballot(cand);
        if (m == 0) return;
        const uint32_t before = __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
        if (cand) stage[count + before] = word;
        count += (uint32_t)__popcll(m);
    }

    __device__ __forceinline__ void drain()
    {
        while (count >= (uint32_t)L) flush();
    }

    // Offer one word per lane (valid lanes only) and merge when L are waiting.
    __device__ __forceinline__ void offer(bool valid, uint64_t word)
    {
        stage_only(valid, word);
        drain();
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
    // column blocks of one wide matrix (KNN): key of a score that k earlier columns of the row reach, 0 = none yet; raised here
    uint32_t* row_bound;        // [batch]
    // guided variant: maxima of the row's 64-column segments, left by the producer of `in`
    const float* seg_max;       // [batch][nseg]
    uint32_t nseg;
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

// End of a (row, segment): merges the lists of the four waves into wave 0 and writes the result (final pairs, or packed words
// for the merge kernel).  Every lane of the workgroup must call it.
template <int R>
__device__ __forceinline__ void finish_row(WaveTopK<R>& list, uint64_t (*sStage)[WaveTopK<R>::kStageWords], const TopKArgs& a,
                                           uint32_t b, uint32_t seg, uint32_t wave, uint32_t lane)
{
    // Merge the four waves into wave 0.  A wave that never had to flush hands over its staged words as they are (they
    // already sit in LDS); a wave with a register list flushes what is left and publishes its first k words.
    __shared__ uint32_t sPublished[kTopkWaves];
    __shared__ uint32_t sFlushed[kTopkWaves];
    __shared__ uint32_t sPlace[2 * kWave];
    if (wave != 0 && list.flushed) {
        list.finish();
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint32_t p = r * kWave + lane;
            if (p < a.k) sStage[wave][p] = list.q[r];
        }
    }
    if (lane == 0) {
        sPublished[wave] = (wave != 0 && list.flushed) ? a.k : list.count;
        sFlushed[wave] = list.flushed ? 1u : 0u;
    }
    if (wave == 1) {
        sPlace[lane] = 0;
        sPlace[kWave + lane] = 0;
    }
    __syncthreads();

    uint64_t* partial = a.partial ? a.partial + ((uint64_t)b * a.partial_slots + a.partial_slot0 + seg) * a.k : nullptr;
    float* keys = a.keys + (uint64_t)b * a.k;
    uint32_t* values = a.values + (uint64_t)b * a.k;
    // result slot p of this (row, segment): a packed word for the merge kernel, or the final (score, column) pair
    auto write_slot = [&](uint32_t p, uint64_t word) {
        float key = -kMaxValue;   // engine/kernels.cu:3221-3224: unfilled slots
        uint32_t col = 0;
        if (word != 0) {
            unpack_score(word, key, col);
            col += a.col_offset;
        }
        if (partial) {
            partial[p] = (word != 0) ? ((word & 0xffffffff00000000ull) | (uint32_t)~col) : 0ull;
        } else {
            keys[p] = key;
            values[p] = col;
        }
    };

    const uint32_t n0 = sPublished[0], n1 = sPublished[1], n2 = sPublished[2], n3 = sPublished[3];
    const uint32_t total = n0 + n1 + n2 + n3;
    const bool any_flushed = (sFlushed[0] | sFlushed[1] | sFlushed[2] | sFlushed[3]) != 0;   // the same for every wave
    if (!any_flushed && total <= 2 * kWave) {
        // Common case for small k: at most 128 staged words in all.  Lane i takes the i-th (and the 64 + i-th) of them; the
        // number of staged words that are larger is its place in the result, so no sorting network runs at all.  The
        // counting is shared: every wave compares all words with its own staged ones and adds its count in LDS.
        auto fetch = [&](uint32_t i) -> uint64_t {
            if (i >= total) return 0ull;   // never larger than anything
            const uint32_t w = (i >= n0) + (i >= n0 + n1) + (i >= n0 + n1 + n2);
            const uint32_t first = (w == 0) ? 0 : (w == 1) ? n0 : (w == 2) ? n0 + n1 : n0 + n1 + n2;
            return sStage[w][i - first];
        };
        const bool two = total > kWave;   // workgroup-uniform
        const uint64_t word0 = fetch(lane), word1 = two ? fetch(kWave + lane) : 0ull;
        const uint32_t mine = sPublished[wave];
        uint32_t part0 = 0, part1 = 0;
        for (uint32_t i = 0; i < mine; i += 4) {   // broadcast reads, four in flight (a staging row has room beyond any count)
            uint64_t o[4];
#pragma unroll
            for (int u = 0; u < 4; u++) o[u] = sStage[wave][i + u];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                if (i + u >= mine) o[u] = 0ull;   // stale words beyond the count
                part0 += (o[u] > word0) ? 1u : 0u;
                if (two) part1 += (o[u] > word1) ? 1u : 0u;
            }
        }
        if (part0 != 0) atomicAdd(&sPlace[lane], part0);
        if (part1 != 0) atomicAdd(&sPlace[kWave + lane], part1);
        __syncthreads();
        if (wave != 0) return;
        const uint32_t place0 = sPlace[lane], place1 = sPlace[kWave + lane];
        if (word0 != 0 && place0 < a.k) write_slot(place0, word0);
        if (word1 != 0 && place1 < a.k) write_slot(place1, word1);
        for (uint32_t p = total + lane; p < a.k; p += kWave) write_slot(p, 0ull);
        if (a.row_bound) {   // this block's k-th score bounds the row's final k-th from below
            if (word0 != 0 && place0 == a.k - 1) atomicMax(&a.row_bound[b], (uint32_t)(word0 >> 32));
            if (word1 != 0 && place1 == a.k - 1) atomicMax(&a.row_bound[b], (uint32_t)(word1 >> 32));
        }
        return;
    }
    if (wave != 0) return;

    for (uint32_t w = 1; w < kTopkWaves; w++) {
        const uint32_t n = sPublished[w];
        for (uint32_t p0 = 0; p0 < n; p0 += kWave) {
            const uint32_t p = p0 + lane;
            uint64_t word = 0;
            if (p < n) word = sStage[w][p];
            list.offer(word != 0, word);
        }
    }
    list.finish();
#pragma unroll
    for (int r = 0; r < R; r++) {
        const uint32_t p = r * kWave + lane;
        if (p < a.k) write_slot(p, list.q[r]);
        if (a.row_bound && p == a.k - 1 && list.q[r] != 0) atomicMax(&a.row_bound[b], (uint32_t)(list.q[r] >> 32));
    }
}

template <int R, bool FILTERED>
__global__ __launch_bounds__(kTopkThreads, (R <= 2) ? 4 : 2) void topk_scan_kernel(TopKArgs a)
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
    if (a.row_bound) {
        const uint32_t t = a.row_bound[b];   // k columns of earlier blocks of this row reach this score
        if (t > score_key(-__builtin_inff())) list.prime(t);
    }

    // Software pipeline: the lane's first 2 * CH 16-byte groups are requested before anything else happens (the filter's
    // chain of dependent loads would otherwise sit in front of the scan), and inside the loop two spans are in flight while
    // one is examined.  Groups beyond the segment are filled with NaN, which fails every comparison below.
    constexpr int CH = 8;
    const float4* body = reinterpret_cast<const float4*>(row + head);
    const uint32_t step = kTopkThreads;
    auto load_span = [&](float4 (&d)[CH], uint32_t first) {   // first: block-uniform group number
        const uint32_t g = first + threadIdx.x;
        if (first + CH * step <= g1) {
#pragma unroll
            for (int u = 0; u < CH; u++) d[u] = body[g + u * step];
        } else {
            const float nan = __uint_as_float(0x7fc00000u);
#pragma unroll
            for (int u = 0; u < CH; u++) {
                d[u] = make_float4(nan, nan, nan, nan);
                if (g + u * step < g1) d[u] = body[g + u * step];
            }
        }
    };
    // the filter's row range first: it heads a chain of dependent loads
    uint64_t fs = 0, fe = 0;
    if constexpr (FILTERED) {
        uint32_t r = a.position + b;
        if (a.index) r = a.index[r];
        fs = a.fstart[r];
        fe = a.fend[r];
    }
    uint32_t span = g0;
    float4 cur[CH], nxt[CH];
    load_span(cur, span);
    // Head (segment 0) and tail (last segment): at most 3 + 3 columns, taken by wave 0 and examined after the scan.
    uint32_t ht_col = 0xffffffffu;
    float ht_val = 0.0f;
    if (wave == 0) {
        if (seg == 0 && lane < head) ht_col = lane;
        if (seg == a.segments - 1 && lane >= 32 && (lane - 32) < a.width - tail0) ht_col = tail0 + (lane - 32);
        if (ht_col != 0xffffffffu) ht_val = row[ht_col];
    }

    // Filter, part one: mark the listed columns in the bitmap, note which lanes hold a listed column in their first CH groups
    // (they sit out the priming below), and request the scores of the first kFU * 256 listed columns.  The listed items
    // themselves are injected after the scan, when the threshold is tight and nearly all of them fail the first compare.
    // Vector loads complete in the order they were issued, so the column numbers are requested between the first and the
    // second span: waiting for them then costs no more than waiting for the first span, which priming needs anyway, and the
    // listed scores (requested last) are not waited for until the scan is over.
    constexpr int kFU = (R >= 2) ? 2 : 4;   // (the longer lists of k > 64 need the registers: fewer listed columns are held at once)
    __shared__ uint32_t sTaint[kTopkThreads / 2];   // 16 bits per lane: bit u = group u of the first two spans holds a listed column
    uint32_t fcol[kFU];
    float fm[kFU], fv[kFU];
    if constexpr (FILTERED) {
#pragma unroll
        for (int u = 0; u < kFU; u++) {
            const uint64_t t = fs + (uint64_t)u * kTopkThreads + threadIdx.x;
            fcol[u] = 0xffffffffu;
            fm[u] = 0.0f;   // utils/Filters.cpp:62 with the default multiplier
            if (t < fe) {
                fcol[u] = a.fidx[t];
                if (a.fmul) fm[u] = a.fmul[t];
            }
        }
    }
    load_span(nxt, span + CH * step);
    if constexpr (FILTERED) {
        const uint32_t words = (hi - lo + 31) / 32;
        for (uint32_t i = threadIdx.x; i < words; i += kTopkThreads) sBitmap[i] = 0;
        if (threadIdx.x < kTopkThreads / 2) sTaint[threadIdx.x] = 0;
        __syncthreads();
        auto mark = [&](uint32_t c) {
            if (c >= lo && c < hi) {
                atomicOr(&sBitmap[(c - lo) >> 5], 1u << ((c - lo) & 31));
                if (c >= head && c < tail0) {
                    const uint32_t gi = (c - head) / 4 - g0;
                    if (gi < 2 * CH * step) atomicOr(&sTaint[(gi % step) >> 1], 1u << (((gi % step) & 1) * 16 + gi / step));
                }
            }
        };
        // With the default multiplier (every listed column is multiplied by 0) the listed scores are only of interest to a
        // wavefront whose k-th score is not above 0 by the end of the scan: they are then read at that point, not up here.
#pragma unroll
        for (int u = 0; u < kFU; u++) {
            fv[u] = 0.0f;
            if (a.fmul && fcol[u] >= lo && fcol[u] < hi) fv[u] = row[fcol[u]];
            mark(fcol[u]);
        }
        for (uint64_t t = fs + (uint64_t)kFU * kTopkThreads + threadIdx.x; t < fe; t += kTopkThreads) mark(a.fidx[t]);
        __syncthreads();
    }

    auto filtered_out = [&](uint32_t col) -> bool {
        if constexpr (FILTERED) {
            return (sBitmap[(col - lo) >> 5] >> ((col - lo) & 31)) & 1u;
        } else {
            return false;
        }
    };

    // Priming (k <= 128): before anything is admitted, every lane takes the best score of its groups in each of the first two spans.
    // The k-th best of a wave's 128 maxima is a score that at least k unfiltered items reach, so nothing below it can be in the
    // result; the k-th best of the 4k scores the four waves publish is a bound for the whole workgroup.  It is found by
    // binary search on the key bits (no sorting), and the scan then admits a few dozen items per row instead of a few
    // hundred.  Groups that hold a listed column are left out, and a lane with nothing else contributes -inf, which only
    // weakens the bound.
    // The two maxima of a lane are those of its groups in the first and in the second span: together the first 2 * CH * 4 KiB of
    // the segment, 60 % of a 27,278-column row.  (A bound from the first span alone admits twice as many items on average
    // and, in the unlucky row of a large batch, ten times as many: the slowest row sets the kernel's time.)
    __shared__ uint32_t sPrime[kTopkWaves][2 * kWave];
    auto prime_from_first_spans = [&]() {
        constexpr int PV = 2;
        uint32_t taint = 0;
        if constexpr (FILTERED) taint = (sTaint[threadIdx.x >> 1] >> ((threadIdx.x & 1) * 16)) & 0xffffu;
        uint32_t key[PV];
#pragma unroll
        for (int v = 0; v < PV; v++) {
            float m = -__builtin_inff();
#pragma unroll
            for (int u = 0; u < CH; u++) {
                const float4& g = (v == 0) ? cur[u] : nxt[u];
                const float gm = fmaxf(fmaxf(g.x, g.y), fmaxf(g.z, g.w));   // fmaxf drops NaN
                m = fmaxf(m, ((taint >> (v * CH + u)) & 1u) ? -__builtin_inff() : gm);
            }
            key[v] = score_key(m);
        }
        const uint32_t tw = wave_kth_key<PV>(key, a.k);
        uint32_t published = 0;   // wave-uniform
#pragma unroll
        for (int v = 0; v < PV; v++) {
            const bool pub = key[v] >= tw;   // at least k values of the wavefront
            const uint64_t pm = __ballot(pub);
            const uint32_t pos = published + __builtin_amdgcn_mbcnt_hi((uint32_t)(pm >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)pm, 0u));
            if (pub && pos < a.k) sPrime[wave][pos] = key[v];
            published += (uint32_t)__popcll(pm);
        }
        __syncthreads();
        uint32_t all[4 * PV];   // the 4k published keys, side by side
#pragma unroll
        for (int n = 0; n < 4 * PV; n++) {
            const uint32_t i = n * kWave + lane;
            all[n] = (i < kTopkWaves * a.k) ? sPrime[i / a.k][i % a.k] : 0u;
        }
        uint32_t t;
        if (a.k <= 16) t = wave_kth_key<1>(reinterpret_cast<const uint32_t(&)[1]>(all), a.k);
        else if (a.k <= 32) t = wave_kth_key<2>(reinterpret_cast<const uint32_t(&)[2]>(all), a.k);
        else if (a.k <= 64) t = wave_kth_key<4>(reinterpret_cast<const uint32_t(&)[4]>(all), a.k);
        else t = wave_kth_key<4 * PV>(all, a.k);
        if (t > score_key(-__builtin_inff())) {
            list.prime(t);
            // Rows whose best scores tie in their hundreds (saturated sigmoids: exactly 1.0f in every eighth column) would
            // otherwise stage every group that holds one of them until a list fills up and is sorted.  Among equal scores the
            // lower column wins, so the bound gets a column: a wavefront's first group is 256 consecutive columns, the lowest it
            // will see; if k of them reach the bound, the k-th such column X closes the bound — a score equal to it passes at or
            // before X only, and every later group fails the one compare of the scan.
            const float S = key_score(t);
            const float4& g = cur[0];
            const float e[4] = {g.x, g.y, g.z, g.w};
            const uint32_t col = head + 4 * (span + threadIdx.x);
            bool ok[4];
            uint32_t before = 0, mine = 0, total = 0;
#pragma unroll
            for (int c = 0; c < 4; c++) {
                ok[c] = e[c] >= S;
                if constexpr (FILTERED) {
                    if (ok[c]) ok[c] = !filtered_out(col + c);
                }
                const uint64_t q = __ballot(ok[c]);
                before += __builtin_amdgcn_mbcnt_hi((uint32_t)(q >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)q, 0u));
                mine += ok[c] ? 1u : 0u;
                total += (uint32_t)__popcll(q);
            }
            if (total >= a.k) {   // wave-uniform
                const bool has = before < a.k && a.k <= before + mine;   // exactly one lane
                uint32_t need = has ? a.k - before : 0u, colX = 0;
#pragma unroll
                for (int c = 0; c < 4; c++)
                    if (ok[c] && need != 0 && --need == 0) colX = col + c;
                const uint64_t hm = __ballot(has);
                const uint32_t X = (uint32_t)__builtin_amdgcn_readlane((int)colX, __builtin_ctzll(hm));
                list.prime_word(pack_score(S, X));
            }
        }
    };
    if (R <= 2 && g0 < g1) prime_from_first_spans();   // (k <= 128)

    // The four scores of one 16-byte group; at most 4 * 64 words are staged.
    auto stage_group = [&](const float4& v, uint32_t col) {
        float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int c = 0; c < 4; c++) {
            asm volatile("" : "+v"(e[c]));   // keeps the packing below inside the (rarely taken) branch instead of hoisted for all groups
            bool ok = e[c] >= list.thr_key;
            if (__ballot(ok) == 0) continue;
            if constexpr (FILTERED) {
                if (ok) ok = !filtered_out(col + c);
            }
            list.stage_only(ok, pack_score(e[c], col + c));
        }
    };
    static_assert(CH == 8, "the scan selects among eight groups");
    static_assert(List::kBurst >= 4 * kWave, "a group stages up to 256 words between drains");

    // Body: the block walks the segment in spans of CH * 4 KiB, wave w takes the w-th KiB of each 4 KiB.  The common case
    // costs three vector instructions per group (maximum of four, one compare); groups with a survivor somewhere in the wave
    // are then walked one at a time.
    while (span < g1) {
        const uint32_t gbase = span + threadIdx.x;
        uint32_t hot = 0;
        {
            const float t = list.admission_score(head + 4 * span);   // every column of this span and after is at or beyond that
            const float t1 = list.admission_score(head + 4 * (span + step));   // ... and every column of its groups 1 to 7 at or beyond this
#pragma unroll
            for (int u = 0; u < CH; u++) {
                const float m = fmaxf(fmaxf(cur[u].x, cur[u].y), fmaxf(cur[u].z, cur[u].w));
                if (__ballot(m >= (u == 0 ? t : t1)) != 0) hot |= 1u << u;
            }
        }
        while (hot != 0) {
            const int u = __ffs(hot) - 1;
            hot &= hot - 1;
            const uint32_t col = head + 4 * (gbase + (uint32_t)u * step);
            switch (u) {
            case 0: stage_group(cur[0], col); break;
            case 1: stage_group(cur[1], col); break;
            case 2: stage_group(cur[2], col); break;
            case 3: stage_group(cur[3], col); break;
            case 4: stage_group(cur[4], col); break;
            case 5: stage_group(cur[5], col); break;
            case 6: stage_group(cur[6], col); break;
            default: stage_group(cur[7], col); break;
            }
            list.drain();
        }
#pragma unroll
        for (int u = 0; u < CH; u++) cur[u] = nxt[u];
        span += CH * step;
        load_span(nxt, span + CH * step);
    }

    // Head and tail columns (requested at the start of the kernel).
    if (wave == 0) {
        const bool ok = (ht_col != 0xffffffffu) && (ht_val >= list.thr_key) && !filtered_out(ht_col);
        list.stage_only(ok, pack_score(ht_val, ht_col));
    }

    // Filter, part two: every listed column is injected once with score * multiplier.  The lane that clears a column's bit
    // owns it (a column listed twice is injected once).  The bitmap is no longer consulted after the barrier.
    if constexpr (FILTERED) {
        __syncthreads();
        // A listed column multiplied by 0 scores 0 (or nothing at all, if its score is not finite): it cannot enter the list of
        // a wavefront that already holds k scores above 0, and the final k-th score is at least that wavefront's.
        const bool zeros_matter = a.fmul != nullptr || !(list.thr_key > 0.0f);   // wave-uniform
        for (uint64_t base = fs; base < fe && zeros_matter; base += (uint64_t)kFU * kTopkThreads) {
            if (base != fs || !a.fmul) {
                if (base != fs) {
#pragma unroll
                    for (int u = 0; u < kFU; u++) {
                        const uint64_t t = base + (uint64_t)u * kTopkThreads + threadIdx.x;
                        fcol[u] = 0xffffffffu;
                        fm[u] = 0.0f;
                        if (t < fe) {
                            fcol[u] = a.fidx[t];
                            if (a.fmul) fm[u] = a.fmul[t];
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < kFU; u++) {
                    fv[u] = 0.0f;
                    if (fcol[u] >= lo && fcol[u] < hi) fv[u] = row[fcol[u]];
                }
            }
#pragma unroll
            for (int u = 0; u < kFU; u++) {
                if (base + (uint64_t)u * kTopkThreads + wave * kWave >= fe) break;   // wave-uniform
                bool own = false;
                if (fcol[u] >= lo && fcol[u] < hi) {
                    const uint32_t bit = 1u << ((fcol[u] - lo) & 31);
                    own = (atomicAnd(&sBitmap[(fcol[u] - lo) >> 5], ~bit) & bit) != 0;
                }
                const float v = fm[u] * fv[u];   // utils/Filters.cpp:62
                list.stage_only(own && v == v, pack_score(v, fcol[u]));   // NaN never enters (it fails every comparison)
            }
            list.drain();
        }
    }

    finish_row<R>(list, sStage, a, b, seg, wave, lane);
}

// Guided top-K (k <= 64): the producer of the scores also left the maximum of every 64-column segment of every row (the
// dense layer's epilogue has them in registers anyway).  The k-th largest of a row's segment maxima is a score that at least
// k items reach, so only segments whose maximum reaches it can hold a result: about k of them.  The kernel reads the
// row's maxima (1/64 of the row), picks that bound with the same key-bit search the scan uses for priming, and then reads
// just those segments.  With the filter, a maximum that is the score of a listed column says nothing about the unlisted
// ones: it is left out of the bound (its segment is still read).  Rows full of ties read more segments and still come out
// right: the survivors go through the same lists as in the scan.
constexpr uint32_t kGuidedSegWidth = 64;
constexpr uint32_t kGuidedMaxSegs = 2048;
constexpr uint32_t kGuidedMaxK = 64;

// E: segment maxima per lane (256 * E >= number of segments); the key search costs in proportion.
template <bool FILTERED, int E>
__global__ __launch_bounds__(kTopkThreads, 4) void topk_guided_kernel(TopKArgs a)
{
    __builtin_amdgcn_s_setprio(3);   // short kernels issue ahead of a GEMM's wavefronts that share their SIMD
    using List = WaveTopK<1>;
    static_assert(E * kTopkThreads <= kGuidedMaxSegs, "at most kGuidedMaxSegs segments");
    __shared__ uint64_t sStage[kTopkWaves][List::kStageWords];
    __shared__ uint32_t sPrime[kTopkWaves][kGuidedMaxK];
    __shared__ uint32_t sListCount, sBound;
    __shared__ uint32_t sChunk[8 * kTopkWaves];   // listed segments per group of 64 maxima
    extern __shared__ uint32_t sDyn[];   // segments to read [nseg] | their maxima [nseg] | best listed score per segment [nseg] | bitmap of listed columns
    uint32_t* sList = sDyn;
    uint32_t* sListKey = sDyn + a.nseg;
    uint32_t* sFiltMax = sDyn + 2 * a.nseg;
    uint32_t* sBitmap = sDyn + 3 * a.nseg;

    const uint32_t b = blockIdx.x;
    const uint32_t wave = threadIdx.x / kWave;
    const uint32_t lane = threadIdx.x % kWave;
    const float* row = a.in + (uint64_t)b * a.pitch;
    List list;
    list.init(sStage[wave], lane, a.k);

    uint64_t fs = 0, fe = 0;
    if constexpr (FILTERED) {
        uint32_t r = a.position + b;
        if (a.index) r = a.index[r];
        fs = a.fstart[r];
        fe = a.fend[r];
    }
    uint32_t mk[E];   // keys of this lane's segment maxima; 0 = no such segment
    {
        const float* mrow = a.seg_max + (uint64_t)b * a.nseg;
#pragma unroll
        for (int e = 0; e < E; e++) {
            const uint32_t idx = e * kTopkThreads + threadIdx.x;
            mk[e] = (idx < a.nseg) ? score_key(mrow[idx]) : 0u;
        }
    }
    sPrime[wave][lane] = 0;
    if (threadIdx.x == 0) sListCount = 0;

    constexpr int kFU = 4;
    uint32_t fcol[kFU];
    float fm[kFU], fv[kFU];
    // A row with few listed columns and the default multiplier does not read their scores at all (one round trip less on the
    // way to the bound): a segment that holds a listed column is simply left out of the bound, and a listed column's zero is
    // only looked at when zeros can still enter a list.  A long list would leave too few segments for a good bound: such rows,
    // and rows with multipliers, read the listed scores first and leave out only the segments whose maximum is one of them.
    bool light = false;   // the same for the whole workgroup
    if constexpr (FILTERED) {
        light = !a.fmul && (fe - fs) * 2 <= a.nseg;
        // (the listed columns are requested before the barrier below, which waits for everything in flight: the row's range,
        // the maxima and the first listed columns then cost two round trips, not three)
#pragma unroll
        for (int u = 0; u < kFU; u++) {
            const uint64_t t = fs + (uint64_t)u * kTopkThreads + threadIdx.x;
            fcol[u] = 0xffffffffu;
            fm[u] = 0.0f;   // utils/Filters.cpp:62 with the default multiplier
            if (t < fe) {
                fcol[u] = a.fidx[t];
                if (a.fmul) fm[u] = a.fmul[t];
            }
        }
        const uint32_t words = (a.width + 31) / 32;
        for (uint32_t i = threadIdx.x; i < words; i += kTopkThreads) sBitmap[i] = 0;
        for (uint32_t i = threadIdx.x; i < a.nseg; i += kTopkThreads) sFiltMax[i] = 0;
        __syncthreads();
        auto mark = [&](uint32_t c, float v) {
            atomicOr(&sBitmap[c >> 5], 1u << (c & 31));
            if (v == v) atomicMax(&sFiltMax[c / kGuidedSegWidth], score_key(v));   // a NaN is never a segment's maximum
        };
        if (light) {   // (at most nseg / 2 <= 1024 listed columns: they are all in fcol)
#pragma unroll
            for (int u = 0; u < kFU; u++) {
                fv[u] = 0.0f;
                if (fcol[u] < a.width) {
                    atomicOr(&sBitmap[fcol[u] >> 5], 1u << (fcol[u] & 31));
                    sFiltMax[fcol[u] / kGuidedSegWidth] = 0xffffffffu;   // equal to no key of a maximum that takes part (NaN patterns aside, which are 0 here)
                }
            }
        } else {
#pragma unroll
            for (int u = 0; u < kFU; u++) {
                fv[u] = 0.0f;
                if (fcol[u] < a.width) fv[u] = row[fcol[u]];
            }
#pragma unroll
            for (int u = 0; u < kFU; u++)
                if (fcol[u] < a.width) mark(fcol[u], fv[u]);
            for (uint64_t t = fs + (uint64_t)kFU * kTopkThreads + threadIdx.x; t < fe; t += kTopkThreads) {
                const uint32_t c = a.fidx[t];
                if (c < a.width) mark(c, row[c]);
            }
        }
    }
    __syncthreads();

    auto filtered_out = [&](uint32_t col) -> bool {
        if constexpr (FILTERED) {
            return (sBitmap[col >> 5] >> (col & 31)) & 1u;
        } else {
            return false;
        }
    };

    // The bound: k-th largest of the maxima that are not a listed column's score, first per wave, then over the 4k the waves
    // publish.  With fewer than k such maxima there is no bound and every segment is read.
    uint32_t bound = 0;
    {
        uint32_t tk[E];
#pragma unroll
        for (int e = 0; e < E; e++) {
            tk[e] = mk[e];
            if constexpr (FILTERED) {
                const uint32_t idx = e * kTopkThreads + threadIdx.x;
                if (idx < a.nseg && (light ? sFiltMax[idx] != 0 : sFiltMax[idx] == mk[e])) tk[e] = 0;
            }
        }
        if (a.k <= 16) {   // the same for the whole workgroup
            // Small k: the maxima go to LDS, one wavefront takes the largest of each lane's share (every 64th) and searches
            // those 64.  The k-th largest of them is reached by k real items as well; it is the exact k-th maximum unless two of
            // the k best share a lane (then it is the next one down, and a segment more is read) — one short search instead of
            // a search per wavefront and a second one over what they publish.
#pragma unroll
            for (int e = 0; e < E; e++) {
                const uint32_t idx = e * kTopkThreads + threadIdx.x;
                if (idx < a.nseg) sListKey[idx] = tk[e];   // (the list of segments is built later)
            }
            __syncthreads();
            if (wave == 0) {
                uint32_t best[1] = {0u};
                for (uint32_t i = lane; i < a.nseg; i += kWave) best[0] = max(best[0], sListKey[i]);
                const uint32_t t = wave_kth_key<1>(best, a.k);
                if (lane == 0) sBound = t;
            }
        } else {
            const uint32_t tw = wave_kth_key<E>(tk, a.k);
            uint32_t published = 0;   // wave-uniform
#pragma unroll
            for (int e = 0; e < E; e++) {
                const bool pub = tk[e] != 0 && tk[e] >= tw;
                const uint64_t pm = __ballot(pub);
                const uint32_t pos = published + __builtin_amdgcn_mbcnt_hi((uint32_t)(pm >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)pm, 0u));
                if (pub && pos < a.k) sPrime[wave][pos] = tk[e];
                published += (uint32_t)__popcll(pm);
            }
            __syncthreads();
            // (one wavefront searches, the others wait: four workgroups share a CU, and what the searches of sixteen wavefronts
            // cost is instruction issue, not latency)
            if (wave == 0) {
                uint32_t all[4];
#pragma unroll
                for (int n = 0; n < 4; n++) {
                    const uint32_t i = n * kWave + lane;
                    all[n] = (i < kTopkWaves * a.k) ? sPrime[i / a.k][i % a.k] : 0u;
                }
                uint32_t t;
                if (a.k <= 32) t = wave_kth_key<2>(reinterpret_cast<const uint32_t(&)[2]>(all), a.k);
                else t = wave_kth_key<4>(all, a.k);
                if (lane == 0) sBound = t;
            }
        }
        __syncthreads();
        const uint32_t t = sBound;
        if (t > score_key(-__builtin_inff())) {
            bound = t;
            list.prime(t);
        }
    }

    // Segments whose maximum (listed or not) reaches the bound.
    uint64_t listed[E];
#pragma unroll
    for (int e = 0; e < E; e++) {
        const uint32_t idx = e * kTopkThreads + threadIdx.x;
        const bool flagged = idx < a.nseg && mk[e] >= bound;
        const uint64_t m = __ballot(flagged);
        listed[e] = m;
        if (m == 0) continue;
        uint32_t base = 0;
        if (lane == 0) base = atomicAdd(&sListCount, (uint32_t)__popcll(m));
        base = (uint32_t)__builtin_amdgcn_readfirstlane((int)base);
        if (flagged) {
            const uint32_t pos = base + __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
            sList[pos] = idx;
            sListKey[pos] = mk[e];
        }
    }
    __syncthreads();
    const uint32_t count = sListCount;
    constexpr int kSegsInFlight = 8;
    // More segments than one round of reads takes (rows of tied scores, mostly): the list is written again in ascending
    // order, so that the first round reads the lowest columns and what only ties behind them can be left out.  Lane j holds
    // the count of the j-th group of 64 maxima; a scan over the first lanes gives every group its place.
    const bool heavy = bound != 0 && count > kTopkWaves * kSegsInFlight;   // the same for the whole workgroup
    if (heavy) {
        if (lane == 0) {
#pragma unroll
            for (int e = 0; e < E; e++) sChunk[e * kTopkWaves + wave] = (uint32_t)__popcll(listed[e]);
        }
        __syncthreads();   // (everyone has read the count and is done with the unordered list)
        const uint32_t mine = (lane < (uint32_t)(E * kTopkWaves)) ? sChunk[lane] : 0u;
        uint32_t incl = mine;
#pragma unroll
        for (int d = 1; d < E * kTopkWaves; d *= 2) {
            const uint32_t up = (uint32_t)__shfl_up((int)incl, d);
            if (lane >= (uint32_t)d) incl += up;
        }
        const uint32_t excl = incl - mine;
#pragma unroll
        for (int e = 0; e < E; e++) {
            const uint32_t base = (uint32_t)__shfl((int)excl, e * kTopkWaves + (int)wave);
            const uint64_t m = listed[e];
            if ((m >> lane) & 1ull) {
                const uint32_t pos = base + __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
                sList[pos] = e * kTopkThreads + threadIdx.x;
                sListKey[pos] = mk[e];
            }
        }
        __syncthreads();
    }

    // One lane per column of a segment, eight segments in flight per wave: the usual dozen or two of segments are one round
    // trip.  A segment whose maximum no longer reaches what its columns need is not read: in a row of saturated scores every
    // segment reaches the bound, but once a wavefront holds k of them, later segments that only tie are out.
    bool first_round = heavy;
    // (the listed segments are dealt out one at a time: the usual dozen or two then keep all four wavefronts busy)
    for (uint32_t i0 = wave; i0 < count; i0 += kTopkWaves * kSegsInFlight) {
        float v[kSegsInFlight];
        uint32_t col[kSegsInFlight];
#pragma unroll
        for (int u = 0; u < kSegsInFlight; u++) {
            v[u] = __uint_as_float(0x7fc00000u);   // NaN fails the compare below
            col[u] = 0;
            const uint32_t i = i0 + u * kTopkWaves;
            if (i < count) {
                const uint32_t first = sList[i] * kGuidedSegWidth;
                if (key_score(sListKey[i]) >= list.admission_score(first)) {   // wave-uniform
                    col[u] = first + lane;
                    if (col[u] < a.width) v[u] = row[col[u]];
                }
            }
        }
        // Rows of tied scores (saturated activations): when the wavefront's first segments already hold k columns that reach
        // the bound, the largest column among the first k of them goes into the bound, and what only ties behind it is
        // neither staged here nor read later.
        if (first_round) {   // wave-uniform
            first_round = false;
            uint64_t qm[kSegsInFlight];   // lanes whose score reaches the bound and whose column is not listed
            uint32_t reach = 0;
#pragma unroll
            for (int u = 0; u < kSegsInFlight; u++) {
                bool q = v[u] >= list.thr_key;
                qm[u] = 0;
                if (__ballot(q) == 0) continue;
                if (q) q = !filtered_out(col[u]);
                qm[u] = __ballot(q);
                reach += (uint32_t)__popcll(qm[u]);
            }
            if (reach >= a.k) {
                const float S = list.thr_key;
                uint32_t need = a.k, X = 0;
                bool found = false;
#pragma unroll
                for (int u = 0; u < kSegsInFlight; u++) {
                    const uint32_t c = (uint32_t)__popcll(qm[u]);
                    if (found || c == 0) continue;
                    int at;
                    if (need > c) {
                        need -= c;
                        at = 63 - __builtin_clzll(qm[u]);
                    } else {
                        const uint32_t rank = __builtin_amdgcn_mbcnt_hi((uint32_t)(qm[u] >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)qm[u], 0u));
                        at = __builtin_ctzll(__ballot(((qm[u] >> lane) & 1ull) && rank + 1 == need));
                        found = true;
                    }
                    const uint32_t x = (uint32_t)__builtin_amdgcn_readlane((int)col[u], at);
                    X = x > X ? x : X;
                }
                list.prime_word(pack_score(S, X));
            }
#pragma unroll
            for (int u = 0; u < kSegsInFlight; u++) {
                if (qm[u] != 0) list.stage_only((qm[u] >> lane) & 1ull, pack_score(v[u], col[u]));
                if ((u & 3) == 3) list.drain();
            }
            list.drain();
            continue;
        }
#pragma unroll
        for (int u = 0; u < kSegsInFlight; u++) {
            bool ok = v[u] >= list.thr_key;
            if (__ballot(ok) == 0) continue;
            if (ok) ok = !filtered_out(col[u]);
            list.stage_only(ok, pack_score(v[u], col[u]));
            if ((u & 3) == 3) list.drain();   // at most four stagings of 64 words between two checks of the fill level
        }
        list.drain();
    }

    // Every listed column is injected once with score * multiplier; the lane that clears a column's bit owns it.  A listed
    // column multiplied by 0 scores 0 (or nothing at all, if its score is not finite): it cannot enter the list of a
    // wavefront that already holds k scores above 0, and the final k-th score is at least that wavefront's.
    if constexpr (FILTERED) {
        __syncthreads();
        const bool zeros_matter = a.fmul != nullptr || !(list.thr_key > 0.0f);   // wave-uniform
        for (uint64_t base = fs; base < fe && zeros_matter; base += (uint64_t)kFU * kTopkThreads) {
            if (base != fs || light) {
                if (base != fs) {
#pragma unroll
                    for (int u = 0; u < kFU; u++) {
                        const uint64_t t = base + (uint64_t)u * kTopkThreads + threadIdx.x;
                        fcol[u] = 0xffffffffu;
                        fm[u] = 0.0f;
                        if (t < fe) {
                            fcol[u] = a.fidx[t];
                            if (a.fmul) fm[u] = a.fmul[t];
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < kFU; u++) {
                    fv[u] = 0.0f;
                    if (fcol[u] < a.width) fv[u] = row[fcol[u]];
                }
            }
#pragma unroll
            for (int u = 0; u < kFU; u++) {
                if (base + (uint64_t)u * kTopkThreads + wave * kWave >= fe) break;   // wave-uniform
                bool own = false;
                if (fcol[u] < a.width) {
                    const uint32_t bit = 1u << (fcol[u] & 31);
                    own = (atomicAnd(&sBitmap[fcol[u] >> 5], ~bit) & bit) != 0;
                }
                const float v = fm[u] * fv[u];   // utils/Filters.cpp:62
                list.stage_only(own && v == v, pack_score(v, fcol[u]));
            }
            list.drain();
        }
    }
    finish_row<1>(list, sStage, a, b, 0, wave, lane);
}

// Second stage: one wavefront per row merges `slots` packed partial lists of k words each.
template <int R>
__global__ __launch_bounds__(kWave) void topk_merge_kernel(const uint64_t* partial, uint32_t slots, uint32_t k, float* keys,
                                                           uint32_t* values)
{
    __builtin_amdgcn_s_setprio(3);   // short kernels issue ahead of a GEMM's wavefronts that share their SIMD
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

static LibScratch g_partial_of[DSX_MAX_LANES];   // per lane: lanes may run a split top-K at the same time

static int ensure_partial(size_t bytes, uint64_t** out)
{
    LibScratch& buf = g_partial_of[current_lane()];
    if (int rc = lib_scratch_reserve(buf, bytes, "top-K partial lists")) return rc;
    *out = static_cast<uint64_t*>(buf.ptr);
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
             uint32_t forced_segments, uint32_t* row_bound, uint64_t* fixed_scratch, size_t fixed_scratch_words)
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
    a.row_bound = row_bound;
    a.segments = forced_segments ? forced_segments : choose_segments(batch, width, filtered);
    if (fixed_scratch && !partial && a.segments > 1 && (size_t)batch * a.segments * k > fixed_scratch_words)
        return set_error(DSX_EINVAL, "top-K: %u rows x %u segments x k = %u need %zu bytes of partial lists, the fixed scratch holds %zu",
                         batch, a.segments, k, (size_t)batch * a.segments * k * sizeof(uint64_t), fixed_scratch_words * sizeof(uint64_t));
    const uint32_t nvec_max = width / 4 + 1;
    const uint32_t gps = (nvec_max + a.segments - 1) / a.segments;
    const size_t bitmap_bytes = filtered ? ((size_t)(4 * gps + 8 + 31) / 32) * 4 + 16 : 0;
    if (partial) {
        a.partial = partial;
        a.partial_slots = partial_slots;
        a.partial_slot0 = partial_slot0;
    } else if (a.segments > 1) {
        uint64_t* lists = fixed_scratch;
        if (!lists) {
            int rc = ensure_partial((size_t)batch * a.segments * k * sizeof(uint64_t), &lists);
            if (rc) return rc;
        }
        a.partial = lists;
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

// Exact KNN with candidate lists: merges a row's running best list (k packed words, best first) with the candidates the last
// column range left behind, writes the best k back, raises the row's bound to their k-th key and empties the candidate
// lists.  One wavefront per row.  The candidates are the row's shared list (cand, cand_count) and, after a sweep
// (knn_f16_sweep_kernel), its `chunks` private lists seg[row][chunk][seg_cap] with fill counts seg_count[row][64].
template <int R>
__global__ __launch_bounds__(kWave) void knn_refresh_kernel(uint64_t* best, const uint64_t* cand, uint32_t* cand_count, uint32_t cap,
                                                            uint32_t k, uint32_t* row_bound, const uint64_t* seg, uint32_t* seg_count,
                                                            uint32_t chunks, uint32_t seg_cap)
{
    using List = WaveTopK<R>;
    __shared__ uint64_t sStage[List::kStageWords];
    __shared__ uint32_t sStart[kWave + 1];
    const uint32_t b = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    List list;
    list.init(sStage, lane, k);
    uint64_t* mine = best + (uint64_t)b * k;
    for (uint32_t p0 = 0; p0 < k; p0 += kWave) {
        const uint32_t p = p0 + lane;
        const uint64_t word = (p < k) ? mine[p] : 0ull;
        list.offer(word != 0, word);
    }
    const uint32_t n = min(cand_count[b], cap);
    const uint64_t* src = cand + (uint64_t)b * cap;
    for (uint32_t p0 = 0; p0 < n; p0 += kWave) {
        const uint32_t p = p0 + lane;
        const uint64_t word = (p < n) ? src[p] : 0ull;
        list.offer(word != 0, word);
    }
    if (seg) {
        // entry e of the chunks' lists laid end to end: lane c holds where chunk c starts
        uint32_t* counts = seg_count + (uint64_t)b * kWave;
        const uint32_t mine_count = (lane < chunks) ? min(counts[lane], seg_cap) : 0u;
        uint32_t incl = mine_count;
#pragma unroll
        for (int d = 1; d < kWave; d *= 2) {
            const uint32_t below = __shfl_up(incl, d);
            if (lane >= (uint32_t)d) incl += below;
        }
        if (lane == 0) sStart[0] = 0;
        sStart[lane + 1] = incl;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        const uint32_t total = sStart[kWave];
        const uint64_t* lists = seg + (uint64_t)b * chunks * seg_cap;
        for (uint32_t e0 = 0; e0 < total; e0 += kWave) {
            const uint32_t e = e0 + lane;
            uint64_t word = 0;
            if (e < total) {
                uint32_t lo = 0, hi = kWave;   // the last chunk that starts at or before e (empty chunks start where the next one does)
                while (hi - lo > 1) {
                    const uint32_t mid = (lo + hi) / 2;
                    if (sStart[mid] <= e) lo = mid;
                    else hi = mid;
                }
                word = lists[(uint64_t)lo * seg_cap + (e - sStart[lo])];
            }
            list.offer(word != 0, word);
        }
        if (lane < chunks) counts[lane] = 0;
    }
    list.finish();
#pragma unroll
    for (int r = 0; r < R; r++) {
        const uint32_t p = r * kWave + lane;
        if (p < k) mine[p] = list.q[r];
        if (p == k - 1 && list.q[r] != 0) row_bound[b] = max(row_bound[b], (uint32_t)(list.q[r] >> 32));
    }
    if (lane == 0) cand_count[b] = 0;
}

int knn_refresh(uint64_t* best, const uint64_t* cand, uint32_t* cand_count, uint32_t cap, uint32_t k, uint32_t* row_bound, uint32_t batch,
                const uint64_t* seg, uint32_t* seg_count, uint32_t chunks, uint32_t seg_cap)
{
    hipStream_t s = ctx().stream;
    if (seg && (chunks == 0 || chunks > (uint32_t)kWave || !seg_count))
        return set_error(DSX_EINVAL, "knn_refresh: %u chunks (1..64)", chunks);
    if (k <= 64)
        hipLaunchKernelGGL((knn_refresh_kernel<1>), dim3(batch), dim3(kWave), 0, s, best, cand, cand_count, cap, k, row_bound, seg, seg_count,
                           chunks, seg_cap);
    else if (k <= 128)
        hipLaunchKernelGGL((knn_refresh_kernel<2>), dim3(batch), dim3(kWave), 0, s, best, cand, cand_count, cap, k, row_bound, seg, seg_count,
                           chunks, seg_cap);
    else
        hipLaunchKernelGGL((knn_refresh_kernel<4>), dim3(batch), dim3(kWave), 0, s, best, cand, cand_count, cap, k, row_bound, seg, seg_count,
                           chunks, seg_cap);
    DSX_LAUNCH_CHECK("knn_refresh_kernel");
    return DSX_OK;
}

// ---------------------------------------------------------------------------------------------------------------------
// Output layer fused with its top-K (dsx_fc_topk): the row's best list so far (k packed words) is merged with the candidates
// the layer's last column range appended, minus the columns the row's filter lists (multiplier 0: the sample's own items).
// One wavefront per row.  The filter is applied by hashing the candidates' columns into an LDS table (at most half full,
// linear probing), striking out every listed column found there, and then offering only the candidates still present.
// A row whose candidate list filled up is flagged; the refresh after the last range recomputes flagged rows from scratch,
// without any list that could fill up: act(bias + x . W) 256 columns at a time (lane = column, k in order), the listed columns
// marked in a bitmap that covers 262,144 columns at a time.  Slow (the whole matrix is read for one row) and exact.
constexpr uint32_t kLayerTableSlots = 8192;   // twice the candidate capacity the layer search uses; as a bitmap: 262,144 columns
constexpr uint32_t kLayerEmpty = 0xffffffffu, kLayerStruck = 0xfffffffeu;   // (no column has these numbers: widths stay below 2^32 - 2)

struct LayerRefreshArgs {
    uint64_t* best;            // [batch][k] packed words, best first, 0 = empty
    const uint64_t* cand;      // [batch][cap]
    uint32_t* cand_count;      // [batch], reset to 0 here
    uint32_t cap;
    uint32_t k;
    uint32_t* row_bound;       // [batch] key of the row's k-th best score, raised here
    uint32_t* row_flag;        // [batch] != 0: the row's list overflowed in this or an earlier range
    uint32_t* flagged_total;   // host-visible word that is set to 1 when a row is flagged (may be NULL)
    uint32_t position;
    const uint32_t* index;
    const uint64_t* fstart;
    const uint64_t* fend;
    const uint32_t* fidx;      // NULL: no filter
    float* keys;               // final range only (else NULL): [batch][k] results
    uint32_t* values;
    // the layer itself, for flagged rows (final range only)
    const float* X;
    const float* W;
    const float* bias;
    uint32_t ldx, ldw, kdim, n;
    uint32_t first_columns;    // columns of the first block, whose listed columns the scanning top-K has dealt with
    uint32_t act;
    float slope, alpha, lambda;
};

__device__ __forceinline__ uint32_t layer_hash(uint32_t col, uint32_t shift) { return (col * 2654435761u) >> shift; }

template <int R>
__device__ __forceinline__ void layer_recompute_row(WaveTopK<R>& list, const LayerRefreshArgs& a, uint32_t b, uint32_t lane, uint64_t fs,
                                                    uint64_t fe, uint32_t* sBits)
{
    constexpr uint32_t kSpan = kLayerTableSlots * 32;
    const float* x = a.X + (uint64_t)b * a.ldx;
    for (uint32_t C0 = 0; C0 < a.n; C0 += kSpan) {
        for (uint32_t i = lane; i < kLayerTableSlots; i += kWave) sBits[i] = 0;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        for (uint64_t t = fs + lane; t < fe; t += kWave) {
            const uint32_t c = a.fidx[t];
            if (c >= C0 && c - C0 < kSpan) atomicOr(&sBits[(c - C0) >> 5], 1u << ((c - C0) & 31));
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        const uint32_t C1 = (a.n - C0 < kSpan) ? a.n : C0 + kSpan;
        for (uint32_t c0 = C0; c0 < C1; c0 += 4 * kWave) {
            float sum[4];
            uint32_t col[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                col[j] = c0 + j * kWave + lane;
                sum[j] = (a.bias && col[j] < C1) ? a.bias[col[j]] : 0.0f;
            }
            for (uint32_t kk = 0; kk < a.kdim; kk++) {
                const float xk = x[kk];
                const float* w = a.W + (uint64_t)kk * a.ldw;
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (col[j] < C1) sum[j] = fmaf(xk, w[col[j]], sum[j]);
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float y = activate_rt(sum[j], a.act, a.slope, a.alpha, a.lambda);
                const uint32_t off = col[j] - C0;
                // a listed column keeps its place with score * 0 (utils/Filters.cpp:62), once however often it is listed
                if (col[j] < C1 && ((sBits[off >> 5] >> (off & 31)) & 1u)) y *= 0.0f;
                list.offer(col[j] < C1 && y == y, pack_score(y, col[j]));
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
}

template <int R>
__global__ __launch_bounds__(kWave) void layer_refresh_kernel(LayerRefreshArgs a)
{
    __builtin_amdgcn_s_setprio(3);   // short kernels issue ahead of a GEMM's wavefronts that share their SIMD
    using List = WaveTopK<R>;
    __shared__ uint64_t sStage[List::kStageWords];
    __shared__ uint32_t sTable[kLayerTableSlots];
    const uint32_t b = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    const uint32_t count = a.cand_count[b];
    bool flagged = a.row_flag[b] != 0;
    __builtin_amdgcn_wave_barrier();
    if (lane == 0) a.cand_count[b] = 0;
    if (!flagged && count > a.cap) {
        flagged = true;
        if (lane == 0) {
            a.row_flag[b] = 1;
            if (a.flagged_total) *(volatile uint32_t*)a.flagged_total = 1u;
        }
    }
    const bool final_range = a.keys != nullptr;
    if (flagged && !final_range) return;
    uint64_t fs = 0, fe = 0;
    if (a.fidx && (count > 0 || flagged || final_range)) {
        uint32_t r = a.position + b;
        if (a.index) r = a.index[r];
        fs = a.fstart[r];
        fe = a.fend[r];
    }
    List list;
    list.init(sStage, lane, a.k);
    if (flagged) {
        layer_recompute_row<R>(list, a, b, lane, fs, fe, sTable);
        list.finish();
        write_final<R>(list.q, lane, a.k, 0, a.keys + (uint64_t)b * a.k, a.values + (uint64_t)b * a.k);
        return;
    }
    const uint64_t* src = a.cand + (uint64_t)b * a.cap;
    const bool filtering = fe > fs && count > 0;   // wave-uniform
    // table size: a power of two, at least twice the candidates
    uint32_t bits = 7;
    while ((1u << bits) < 2 * count) bits++;
    const uint32_t mask = (1u << bits) - 1, shift = 32 - bits;
    if (filtering) {
        for (uint32_t i = lane; i <= mask; i += kWave) sTable[i] = kLayerEmpty;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        for (uint32_t p = lane; p < count; p += kWave) {
            const uint32_t col = ~(uint32_t)src[p];
            uint32_t h = layer_hash(col, shift);
            while (atomicCAS(&sTable[h], kLayerEmpty, col) != kLayerEmpty) h = (h + 1) & mask;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        for (uint64_t t = fs + lane; t < fe; t += kWave) {
            const uint32_t col = a.fidx[t];
            uint32_t h = layer_hash(col, shift);
            for (;;) {
                const uint32_t v = sTable[h];
                if (v == kLayerEmpty) break;
                if (v == col) {
                    sTable[h] = kLayerStruck;
                    break;
                }
                h = (h + 1) & mask;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    uint64_t* mine = a.best + (uint64_t)b * a.k;
    for (uint32_t p0 = 0; p0 < a.k; p0 += kWave) {
        const uint32_t p = p0 + lane;
        const uint64_t word = (p < a.k) ? mine[p] : 0ull;
        list.offer(word != 0, word);
    }
    for (uint32_t p0 = 0; p0 < count; p0 += kWave) {
        const uint32_t p = p0 + lane;
        const uint64_t word = (p < count) ? src[p] : 0ull;
        bool live = word != 0;
        if (filtering && live) {
            const uint32_t col = ~(uint32_t)word;
            uint32_t h = layer_hash(col, shift);
            for (;;) {
                const uint32_t v = sTable[h];
                if (v == col) break;
                if (v == kLayerEmpty) {   // struck out: the chain ends without the column
                    live = false;
                    break;
                }
                h = (h + 1) & mask;
            }
        }
        list.offer(live, word);
    }
    list.finish();
    if (final_range) {
        // The listed columns beyond the first block were struck out above, but a listed column scores 0, not nothing
        // (utils/Filters.cpp:62 multiplies, kCalculateTopK then sees the zero): when the row's k-th score is not above 0, or the
        // row has fewer than k scores, such a zero belongs in the result.  Those rows are computed again, column by column.
        uint64_t kth = 0;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint64_t w = shfl_u64(list.q[r], (int)((a.k - 1) & (kWave - 1)));
            if ((int)((a.k - 1) / kWave) == r) kth = w;
        }
        bool zeros_matter = false;
        if (fe > fs && (kth == 0 || (uint32_t)(kth >> 32) <= score_key(0.0f))) {
            bool beyond = false;
            for (uint64_t t = fs + lane; t < fe; t += kWave) {
                const uint32_t col = a.fidx[t];
                beyond |= col >= a.first_columns && col < a.n;
            }
            zeros_matter = __ballot(beyond) != 0;
        }
        if (zeros_matter) {
            if (lane == 0 && a.flagged_total) *(volatile uint32_t*)a.flagged_total = 1u;
            __builtin_amdgcn_wave_barrier();
            list.init(sStage, lane, a.k);
            layer_recompute_row<R>(list, a, b, lane, fs, fe, sTable);
            list.finish();
        }
        write_final<R>(list.q, lane, a.k, 0, a.keys + (uint64_t)b * a.k, a.values + (uint64_t)b * a.k);
        return;
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const uint32_t p = r * kWave + lane;
        if (p < a.k) mine[p] = list.q[r];
        if (p == a.k - 1 && list.q[r] != 0) a.row_bound[b] = max(a.row_bound[b], (uint32_t)(list.q[r] >> 32));
    }
}

int layer_refresh_run(const LayerRefresh& r, uint32_t batch)
{
    if (2 * r.cap > kLayerTableSlots) return set_error(DSX_EINVAL, "layer_refresh: candidate capacity %u exceeds %u", r.cap, kLayerTableSlots / 2);
    LayerRefreshArgs a{};
    a.best = r.best; a.cand = r.cand; a.cand_count = r.cand_count; a.cap = r.cap; a.k = r.k;
    a.row_bound = r.row_bound; a.row_flag = r.row_flag; a.flagged_total = r.flagged_total;
    a.position = r.position; a.index = r.index; a.fstart = r.fstart; a.fend = r.fend; a.fidx = r.fidx;
    a.keys = r.keys; a.values = r.values;
    a.X = r.X; a.W = r.W; a.bias = r.bias; a.ldx = r.ldx; a.ldw = r.ldw; a.kdim = r.kdim; a.n = r.n;
    a.first_columns = r.first_columns;
    a.act = r.act; a.slope = r.slope; a.alpha = r.alpha; a.lambda = r.lambda;
    hipStream_t s = ctx().stream;
    if (a.k <= 64) hipLaunchKernelGGL((layer_refresh_kernel<1>), dim3(batch), dim3(kWave), 0, s, a);
    else if (a.k <= 128) hipLaunchKernelGGL((layer_refresh_kernel<2>), dim3(batch), dim3(kWave), 0, s, a);
    else hipLaunchKernelGGL((layer_refresh_kernel<4>), dim3(batch), dim3(kWave), 0, s, a);
    DSX_LAUNCH_CHECK("layer_refresh_kernel");
    return DSX_OK;
}

// Guided top-K when it applies (k <= 64, 64-column segments, at most kGuidedMaxSegs of them), the scan otherwise.
int topk_guided_run(const float* in, uint32_t width, uint32_t batch, uint32_t k, float* keys, uint32_t* values, const float* seg_max,
                    uint32_t seg_width, uint32_t position, const uint32_t* index, const uint64_t* fstart, const uint64_t* fend,
                    const uint32_t* fidx, const float* fmul)
{
    const bool filtered = fidx != nullptr;
    const uint32_t nseg = (width + kGuidedSegWidth - 1) / kGuidedSegWidth;
    size_t lds = (size_t)nseg * 8;
    if (filtered) lds += (size_t)nseg * 4 + ((size_t)(width + 31) / 32) * 4;
    if (!seg_max || seg_width != kGuidedSegWidth || k > kGuidedMaxK || nseg > kGuidedMaxSegs || lds > 40 * 1024)
        return topk_run(in, width, width, batch, k, keys, values, position, index, fstart, fend, fidx, fmul, 0, nullptr, 0, 0, 0);
    TopKArgs a{};
    a.in = in;
    a.pitch = width;
    a.width = width;
    a.k = k;
    a.segments = 1;
    a.position = position;
    a.index = index;
    a.fstart = fstart;
    a.fend = fend;
    a.fidx = fidx;
    a.fmul = fmul;
    a.keys = keys;
    a.values = values;
    a.seg_max = seg_max;
    a.nseg = nseg;
#define DSX_GUIDED(F, E) hipLaunchKernelGGL((topk_guided_kernel<F, E>), dim3(batch), dim3(kTopkThreads), lds, ctx().stream, a)
    if (nseg <= 2 * kTopkThreads) {
        if (filtered) DSX_GUIDED(true, 2); else DSX_GUIDED(false, 2);
    } else if (nseg <= 4 * kTopkThreads) {
        if (filtered) DSX_GUIDED(true, 4); else DSX_GUIDED(false, 4);
    } else {
        if (filtered) DSX_GUIDED(true, 8); else DSX_GUIDED(false, 8);
    }
#undef DSX_GUIDED
    DSX_LAUNCH_CHECK("topk_guided_kernel");
    return DSX_OK;
}

// Fixed scratch of dsx_topk_filtered_static: the packed partial lists of rows split over several workgroups,
// [batch][segments][k] words.  Every device the library runs on holds its own copy of the array at its own address; host code
// must use the address hipGetSymbolAddress reports for the current device, never the array's name.
constexpr size_t kStaticScratchWords = (size_t)1 << 21;   // 16 MiB
static __device__ __align__(256) uint64_t scratch[kStaticScratchWords];
constexpr int kStaticMaxDevices = 64;
static uint64_t* g_static_scratch[kStaticMaxDevices] = {};

int topk_static_setup(int device)
{
    if (device < 0 || device >= kStaticMaxDevices) return set_error(DSX_EINVAL, "dsx_init: device %d is beyond the %d this library keeps scratch for", device, kStaticMaxDevices);
    if (g_static_scratch[device]) return DSX_OK;
    void* p = nullptr;
    DSX_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return set_error(DSX_EHIP, "dsx_init: the fixed top-K scratch has no device address");
    g_static_scratch[device] = static_cast<uint64_t*>(p);
    return DSX_OK;
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

int dsx_topk_filtered_static(const float* in, float* keys, uint32_t* values, uint32_t batch, uint32_t width, uint32_t k, uint32_t position,
                             const uint32_t* index, const uint64_t* filter_start, const uint64_t* filter_end,
                             const uint32_t* filter_index, const float* filter_mul)
{
    DSX_REQUIRE_INIT();
    int rc = check_topk("dsx_topk_filtered_static", in, keys, values, width, k);
    if (rc) return rc;
    DSX_CHECK_ARG(!filter_index || (filter_start && filter_end), "dsx_topk_filtered_static: filter_index without filter_start / filter_end");
    uint64_t* lists = g_static_scratch[ctx().device];
    if (!lists) return set_error(DSX_ENOTINIT, "dsx_topk_filtered_static: no scratch address for device %d", ctx().device);
    if (batch == 0) return DSX_OK;
    // Every (row, segment) workgroup writes all k words of its list before the merge reads them: nothing in the scratch has
    // to start at zero, whatever the previous call left there.
    return topk_run(in, width, width, batch, k, keys, values, position, index, filter_start, filter_end, filter_index, filter_mul, 0,
                    nullptr, 0, 0, 0, nullptr, lists, kStaticScratchWords);
}

int dsx_topk_guided(const float* in, float* keys, uint32_t* values, uint32_t batch, uint32_t width, uint32_t k, const float* seg_max,
                    uint32_t seg_width, uint32_t position, const uint32_t* index, const uint64_t* filter_start,
                    const uint64_t* filter_end, const uint32_t* filter_index, const float* filter_mul)
{
    DSX_REQUIRE_INIT();
    int rc = check_topk("dsx_topk_guided", in, keys, values, width, k);
    if (rc) return rc;
    DSX_CHECK_ARG(!filter_index || (filter_start && filter_end), "dsx_topk_guided: filter_index without filter_start / filter_end");
    if (batch == 0) return DSX_OK;
    return topk_guided_run(in, width, batch, k, keys, values, seg_max, seg_width, position, index, filter_start, filter_end,
                           filter_index, filter_mul);
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
