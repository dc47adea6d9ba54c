/*
 * dsx.h — C ABI of libdsx_hip.so: the MI355X (gfx950) device layer under the DSSTNE inference classes.
 *
 * Plain pointers and sizes only.  Every pointer named "device" is an address in HBM obtained from dsx_malloc (or any
 * other HIP allocation of the same process).  All functions return 0 on success and a negative DSX_E* code on failure;
 * dsx_last_error() then returns a message for the calling thread.  Kernels are enqueued on a library-owned HIP stream
 * (created non-blocking: work on the null stream is NOT ordered against it) and return without waiting; dsx_sync() (or any
 * dsx_memcpy_d2h) waits for them.  A caller that touches device memory with its own kernels or copies calls dsx_sync (or
 * dsx_sync_lane) first.
 *
 * Thread safety: like the reference's GpuContext, the library keeps one context per process (selected lane, staging ring,
 * scratch buffers) without locks around it; calls must come from one thread at a time.  Only dsx_last_error is per thread.
 *
 * Each entry point cites the function of the reference (paths relative to the reference root,
 * engine/ = src/amazon/dsstne/engine/, knn/ = src/amazon/dsstne/knn/, utils/ = src/amazon/dsstne/utils/)
 * whose device work it replaces.
 */
#ifndef DSX_H
#define DSX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    DSX_OK = 0,
    DSX_EINVAL = -1,     /* bad argument (null pointer, k out of range, unsupported type, ...) */
    DSX_EHIP = -2,       /* a HIP runtime call failed */
    DSX_ENOTINIT = -3,   /* dsx_init has not been called */
    DSX_ENOMEM = -4,
    DSX_EUNSUPPORTED = -5
};

/* NNDataSetEnums::Attributes bits, engine/NNEnum.h:9-19 */
enum {
    DSX_ATTR_SPARSE = 1,
    DSX_ATTR_BOOLEAN = 2,
    DSX_ATTR_INDEXED = 64,
    DSX_ATTR_WEIGHTED = 128
};

/* NNDataSetEnums::DataType ordinals, engine/NNEnum.h:35-47 */
enum {
    DSX_T_UINT = 0,
    DSX_T_INT = 1,
    DSX_T_LLINT = 2,
    DSX_T_ULLINT = 3,
    DSX_T_FLOAT = 4,
    DSX_T_DOUBLE = 5,
    DSX_T_RGB8 = 6,
    DSX_T_RGB16 = 7,
    DSX_T_UCHAR = 8,
    DSX_T_CHAR = 9
};

/* Activation ordinals, engine/NNTypes.h:91-105 */
enum {
    DSX_ACT_SIGMOID = 0,
    DSX_ACT_TANH = 1,
    DSX_ACT_RELU = 2,
    DSX_ACT_LINEAR = 3,
    DSX_ACT_PRELU = 4,
    DSX_ACT_SOFTPLUS = 5,
    DSX_ACT_SOFTSIGN = 6,
    DSX_ACT_SOFTMAX = 7,
    DSX_ACT_RELUMAX = 8,
    DSX_ACT_LINEARMAX = 9,
    DSX_ACT_ELU = 10,
    DSX_ACT_LRELU = 11,
    DSX_ACT_SELU = 12
};

/* Parameters of the parametric activations (NNLayer::_RELUSlope, _ELUAlpha, _SELULambda, engine/NNLayer.h:157-159). */
typedef struct dsx_act_params {
    float slope;
    float alpha;
    float lambda;
} dsx_act_params;

typedef struct dsx_device_info {
    char name[256];
    char arch[64];
    int compute_units;
    int wavefront_size;
    int lds_bytes_per_cu;
    size_t hbm_bytes;
    size_t hbm_free_bytes;
    int clock_khz;
    int memory_clock_khz;
} dsx_device_info;

/* ---- context: GpuContext::Startup / Shutdown (engine/GpuTypes.cpp:62-406, 434-472) ------------------------------ */
/* dsx_init may be called more than once (same device); the context lives until the matching number of dsx_shutdown calls. */
int dsx_init(int device);
int dsx_shutdown(void);
int dsx_is_initialized(void);
const char* dsx_last_error(void);
int dsx_get_device_info(dsx_device_info* info);
/* GpuContext::GetMemoryUsage (engine/GpuTypes.cpp:520-525): KiB held through dsx_malloc* by this process. */
int dsx_get_memory_usage(int* gpu_kib, int* cpu_kib);
/* The HIP stream (hipStream_t) every kernel of this library is enqueued on, as an opaque pointer. */
void* dsx_stream(void);

/* ---- GpuBuffer<T> storage (engine/GpuTypes.h:392-625) ------------------------------------------------------------ */
/* Device allocation, zero-filled like the GpuBuffer constructor (engine/GpuTypes.h:523). */
int dsx_malloc(void** device_ptr, size_t bytes);
/* Managed allocation (GpuBuffer bManaged = true): host-dereferenceable, zero-filled. */
int dsx_malloc_managed(void** ptr, size_t bytes);
/* Pinned host allocation for staging. */
int dsx_malloc_host(void** host_ptr, size_t bytes);
int dsx_free(void* device_ptr);
int dsx_free_host(void* host_ptr);
int dsx_memset(void* device_ptr, int value, size_t bytes);
/* GpuBuffer::Upload.  host_src may be reused as soon as the call returns; the copy itself is ordered on the library's stream
 * before everything queued later (uploads of up to 4 MiB are staged in pinned memory and not waited for). */
int dsx_memcpy_h2d(void* device_dst, const void* host_src, size_t bytes);
int dsx_memcpy_d2h(void* host_dst, const void* device_src, size_t bytes);   /* GpuBuffer::Download */
int dsx_memcpy_d2d(void* device_dst, const void* device_src, size_t bytes); /* GpuBuffer::Copy     */
int dsx_sync(void);                                                          /* waits for every lane */
/* No counterpart in the reference (which runs everything on the default stream with blocking copies): the library has up to
 * DSX_MAX_LANES lanes, each an in-order stream; whatever is launched goes to the selected one (lane 0 until told otherwise;
 * a lane's stream is made when the lane is first selected).  Batches issued on different lanes run concurrently; uploads,
 * clears, device-to-device copies and timers order all lanes around themselves, dsx_memcpy_d2h and dsx_sync wait for all of
 * them, dsx_memcpy_d2h_lane for one lane only. */
#define DSX_MAX_LANES 4
int dsx_set_lane(int lane);
int dsx_get_lane(void);
int dsx_sync_lane(int lane);   /* waits for everything queued on one lane (a lane never selected: on the selected one) */
int dsx_memcpy_d2h_lane(int lane, void* host_dst, const void* device_src, size_t bytes);
/* For data that arrives batch by batch (no counterpart in the reference, whose uploads block).  dsx_memcpy_h2d_unordered is
 * dsx_memcpy_h2d on the selected lane only: the other lanes are neither waited for nor told to wait, so the copy overlaps with
 * whatever they run.  The caller guarantees that nothing queued on another lane touches device_dst, and calls
 * dsx_lane_wait_other (the selected lane waits for everything queued so far on the other ones) before work on one lane
 * depends on what another lane wrote. */
int dsx_memcpy_h2d_unordered(void* device_dst, const void* host_src, size_t bytes);
/* Several arrays in one call (a batch's CSR arrays): what dsx_memcpy_h2d_unordered would do for each, with the small ones
 * sharing a launch and the host staging one piece while the device copies the one before. */
int dsx_memcpy_h2d_unordered_many(int count, void* const* device_dst, const void* const* host_src, const size_t* bytes);
int dsx_lane_wait_other(void);
/* A marker is a point in the selected lane's queue (no counterpart in the reference): dsx_marker_record places it after
 * everything queued so far on that lane, dsx_marker_wait blocks the calling host thread until the device has passed it (at
 * once for a marker never recorded).  A caller that streams batches uses it to stay a bounded number of batches ahead of the
 * device. */
int dsx_marker_create(void** marker);
int dsx_marker_record(void* marker);
int dsx_marker_wait(void* marker);
int dsx_marker_destroy(void* marker);
/* Two downloads, one wait (no counterpart in the reference, which copies scores and indexes one after the other). */
int dsx_memcpy_d2h_pair(void* host_dst0, const void* device_src0, size_t bytes0, void* host_dst1, const void* device_src1, size_t bytes1);

/* Event timing on the library stream (the reference keeps cudaEvent timings for KNN, knn/KnnExactGpu.cu:130-148). */
int dsx_timer_start(void);
int dsx_timer_stop(float* elapsed_ms); /* records the stop event, waits for it, returns the elapsed milliseconds */

/* ---- layer input --------------------------------------------------------------------------------------------------- */
/* kClearUnit / kClearDualSourceUnit / kClearTripleSourceUnit / kClearQuadSourceUnit (engine/kernels.cu:61-145):
 * unit[b][j] = sum of the nbias (0..4) bias vectors; nbias == 0 zero-fills (engine/NNLayer.cpp:1002-1039). */
int dsx_clear_unit(float* unit, const float* bias0, const float* bias1, const float* bias2, const float* bias3, uint32_t nbias,
                   uint32_t stride, uint32_t batch);

/* kLoadInputUnit<T> / kLoadIndexedInputUnit<T> (engine/kernels.cu:439-562): dense rows -> fp32 unit buffer.
 * index == NULL for un-indexed data. */
int dsx_load_input_unit(uint32_t data_type, uint32_t position, uint32_t batch, uint32_t stride, float* unit, const uint32_t* index,
                        const void* data);

/* kLoadSparseInputUnit / kLoadIndexedSparseInputUnit / kLoadSparseAnalogInputUnit<T> / kLoadIndexedSparseAnalogInputUnit<T>
 * (engine/kernels.cu:147-286): zero-fill then scatter; used when the dataset is too dense for the sparse-Z path. */
int dsx_load_sparse_input_unit(uint32_t attributes, uint32_t data_type, uint32_t position, uint32_t batch, uint32_t stride,
                               float* unit, const uint32_t* index, const uint64_t* sparse_start, const uint64_t* sparse_end,
                               const uint32_t* sparse_index, const float* data_weight, const void* sparse_data);

/* kCalculateSparseZ / kCalculateIndexedSparseZ / kCalculateSparseAnalogZ<T> / kCalculateIndexedSparseAnalogZ<T>
 * (engine/kernels.cu:662-1299; dispatch NNDataSet<T>::CalculateSparseZ, engine/NNTypes.h:527-545):
 *   unit[b][:] = beta * unit[b][:] + sum over the non-zeros t of row r of (w_r * value_t) * weight[sparse_index[t]][:]
 * with r = position + b, or index[position + b] when DSX_ATTR_INDEXED is set; value_t = 1 when DSX_ATTR_BOOLEAN is set;
 * w_r = data_weight[r] when DSX_ATTR_WEIGHTED is set, else 1.  weight is [input width][stride] row-major.
 * A row without non-zeros leaves unit[b] untouched. */
int dsx_sparse_z(uint32_t attributes, uint32_t data_type, uint32_t position, uint32_t batch, uint32_t stride, const float* weight,
                 const uint32_t* index, const uint64_t* sparse_start, const uint64_t* sparse_end, const uint32_t* sparse_index,
                 const float* data_weight, const void* sparse_data, float* unit, float beta);

/* Fused first layer for a layer whose only incoming source is a fast-sparse input:
 * kClearUnit + kCalculate*SparseZ(beta = 1) + CalculateActivation of NNLayer::ForwardPropagateFullyConnected
 * (engine/NNLayer.cpp:994-1167) in one kernel: unit[b][:] = act(bias[:] + sum ...).  bias may be NULL (zero). */
int dsx_sparse_layer_forward(uint32_t attributes, uint32_t data_type, uint32_t position, uint32_t batch, uint32_t stride,
                             const float* weight, const uint32_t* index, const uint64_t* sparse_start, const uint64_t* sparse_end,
                             const uint32_t* sparse_index, const float* data_weight, const void* sparse_data, const float* bias,
                             uint32_t activation, const dsx_act_params* params, float* unit);

/* ---- fully connected layers ------------------------------------------------------------------------------------------ */
/* Forward GEMM of NNLayer::ForwardPropagateFullyConnected (cublasSgemm call, engine/NNLayer.cpp:1056-1096), with the
 * bias initialisation (kClearUnit, :1002-1039) and CalculateActivation (:1157, :1646-1683) optionally fused:
 *   Z[b][j] = act( (accumulate ? Z[b][j] : 0) + bias[j] + sum_k X[b][k] * W[k][j] )
 * X is [batch x k] row-major with row pitch ldx, Z is [batch x n] with row pitch ldz, W is [k x n] row-major
 * (or [n x k] when transposed != 0: shared transposed weights, engine/NNLayer.cpp:1065-1072).
 * bias may be NULL.  activation = DSX_ACT_LINEAR leaves the pre-activation in Z (for layers with several sources). */
int dsx_fc_forward(const float* X, uint32_t ldx, const float* W, int transposed, const float* bias, float* Z, uint32_t ldz,
                   uint32_t batch, uint32_t k, uint32_t n, int accumulate, uint32_t activation, const dsx_act_params* params);

/* dsx_fc_forward that also leaves, for a later top-K over Z, the maximum of every 64-column segment of every row of the
 * activated result: seg_max[b][s] = max over columns 64 s .. 64 s + 63 (< n) of Z[b][.], row pitch ceil(n / 64).  The epilogue
 * of the wide-layer kernel has these values in registers; other shapes leave seg_max untouched and set *seg_width = 0,
 * otherwise *seg_width = 64.  No counterpart in the reference (it is the by-product that lets dsx_topk_guided skip most of
 * the score matrix the reference's kCalculateTopK, engine/kernels.cu:3202-3989, reads in full). */
int dsx_fc_forward_segmax(const float* X, uint32_t ldx, const float* W, int transposed, const float* bias, float* Z, uint32_t ldz,
                          uint32_t batch, uint32_t k, uint32_t n, uint32_t activation, const dsx_act_params* params, float* seg_max,
                          uint32_t* seg_width);

/* The same layer with every fp32 product formed from bf16 matrix instructions: a mode the caller asks for, with no counterpart
 * in the reference (whose cublasSgemm, engine/NNLayer.cpp:1056-1096, multiplies in fp32, as dsx_fc_forward does).  An fp32
 * value is the exact sum of three bf16 values; six of the nine products of two such sums, accumulated in fp32, carry
 * everything above 2^-25 of the full product, so the sums are as close to the exact ones as dsx_fc_forward's (the tests
 * compare both with fp64), at 12 instead of 32 matrix-core cycles per k.  They are not bit-identical to dsx_fc_forward's.
 *
 * Operands are passed pre-split.  dsx_fc_split writes the planes of `rows` vectors of k values each:
 *   k_major == 0: vector r is src[r * ld + 0 .. k)        (X, a [batch x k] unit buffer; W stored [n x k], i.e. transposed)
 *   k_major != 0: vector r is src[0 .. k) * ld + r         (W stored [k x n])
 * into `planes`, dsx_fc_split_bytes(rows, k) bytes of 16-byte aligned device memory (3 x 2 bytes per value, rows padded to
 * 256 and k to 16).  Weights are split once, a layer's input once per batch.  Non-finite operands: an Inf or NaN stays in the
 * first plane, the other planes hold 0, and the six-term sum then contains Inf x 0 and infinities of either sign: a sum with an
 * Inf operand comes out NaN (sometimes +/-Inf) where dsx_fc_forward gives +/-Inf (the candidate modes drop NaN scores), one with a
 * NaN operand NaN as there.  Sums without such
 * an operand are not affected.  Finite values from 3.0e38 up are kept to bf16 precision only.
 * dsx_fc_forward_split then computes Z as dsx_fc_forward (accumulate, bias, activation) and, with seg_max / seg_width non-NULL
 * and accumulate == 0, the segment maxima as dsx_fc_forward_segmax (*seg_width = 64 for every shape).  A plane (2 bytes x rows
 * padded x k padded) must stay below 4 GiB.
 * A workgroup's tile has 128 rows, or 256 for k >= 512 when that still leaves four tiles per compute unit; results do not
 * depend on it. */
uint64_t dsx_fc_split_bytes(uint32_t rows, uint32_t k);
/* dsx_fc_forward (accumulate == 0) that leaves its result a second time as planes: z_planes as dsx_fc_split(Z, ldz, 0, batch, n,
 * z_planes) would write them (dsx_fc_split_bytes(batch, n) bytes), for the layer that takes Z as its input in this mode.  The
 * small-layer kernel (k = 128 or 256, batch x n <= 2^20) writes them itself; every other shape runs the splitter behind the layer. */
int dsx_fc_forward_planes(const float* X, uint32_t ldx, const float* W, int transposed, const float* bias, float* Z, uint32_t ldz,
                          uint32_t batch, uint32_t k, uint32_t n, uint32_t activation, const dsx_act_params* params, void* z_planes);
int dsx_fc_split(const float* src, uint32_t ld, int k_major, uint32_t rows, uint32_t k, void* planes);
int dsx_fc_forward_split(const void* x_planes, const void* w_planes, const float* bias, float* Z, uint32_t ldz, uint32_t batch, uint32_t k,
                         uint32_t n, int accumulate, uint32_t activation, const dsx_act_params* params, float* seg_max,
                         uint32_t* seg_width);

/* kCalculateSigmoidActivation ... kCalculateSELUActivation (engine/kActivation.cu:46-153) and
 * kCalculateSoftMaxActivation (engine/kActivation.cu:155-236), in place on a [batch x stride] buffer. */
int dsx_activation(float* unit, uint32_t batch, uint32_t stride, uint32_t activation, const dsx_act_params* params);

/* kAddBuffers (engine/kernels.cu:4763-4781): dst += src (skip connections, engine/NNLayer.cpp:1099-1103). */
int dsx_add_buffers(float* dst, const float* src, uint64_t size);

/* ---- top-K ----------------------------------------------------------------------------------------------------------- */
/* kCalculateTopK(pOutput, pKey, pValue, batch, width, k) (engine/kernels.cu:3202-3989): per row of `in`
 * ([batch x width], pitch = width) the k largest values, descending, with their column numbers.
 * Order is total: value descending, then column ascending.  1 <= k <= 256.  Slots beyond `width` candidates hold
 * key -999999999999999.0f and index 0 (engine/NNTypes.h:49, engine/kernels.cu:3221-3224). */
int dsx_topk(const float* in, float* keys, uint32_t* values, uint32_t batch, uint32_t width, uint32_t k);

/* kCalculateTopK(pOutputKey, pOutputValue, pKey, pValue, ...) with float payload (engine/kernels.cu:3992-4188) and
 * with uint32 payload (engine/kernels.cu:4190-4385): top-k of (key, value) pairs by key. */
int dsx_topk_kv_f32(const float* in_keys, const float* in_values, float* keys, float* values, uint32_t batch, uint32_t width,
                    uint32_t k);
int dsx_topk_kv_u32(const float* in_keys, const uint32_t* in_values, float* keys, uint32_t* values, uint32_t batch, uint32_t width,
                    uint32_t k);

/* KNN variant kCalculateTopK(out, key, value, batch, width, widthPadding, k) (knn/topk.cu:29-229, knn/topk.h:73):
 * rows have pitch `width`; only the first width - width_padding columns are candidates. */
int dsx_knn_topk(const float* in, float* keys, uint32_t* values, uint32_t batch, uint32_t width, uint32_t width_padding, uint32_t k);

/* Filtered recommendations of NNRecsGenerator::generateRecs (utils/NNRecsGenerator.cpp:132-150): the reference copies
 * the output rows to the host, multiplies score[idx] by the filter value of every (idx, value) entry of the sample's
 * filter (AbstractFilter::updateRecords, utils/Filters.cpp:49-67), uploads and runs kCalculateTopK.  Here the filter is
 * applied on the fly while scanning, `in` is not modified.  The filter of batch row b is CSR row r = position + b
 * (index[position + b] if index != NULL) of (filter_start, filter_end, filter_index, filter_mul); filter_mul == NULL
 * means every multiplier is 0 (utils/Filters.cpp:108-121).  Indexes outside [0, width) are ignored; an index listed
 * more than once in a row is applied once.  Passing a sample's own sparse input arrays drops the items already
 * present in the input. */
int dsx_topk_filtered(const float* in, float* keys, uint32_t* values, uint32_t batch, uint32_t width, uint32_t k, uint32_t position,
                      const uint32_t* index, const uint64_t* filter_start, const uint64_t* filter_end, const uint32_t* filter_index,
                      const float* filter_mul);

/* dsx_topk_filtered (filter_index == NULL: unfiltered, as dsx_topk) for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  The call allocates and
 * frees nothing: the packed partial lists of rows that are split over several workgroups (small batches, or filtered rows
 * wider than 262,080 columns) go to a fixed 16 MiB array in device memory that every GPU the library runs on holds until the
 * process ends.  Rows are split as in dsx_topk_filtered: s = ceil(4 x compute units / batch) workgroups per row when the batch
 * alone does not fill the device (at most width / 8192), and at least ceil(width / 262,080) with a filter.  When
 * batch x s x k exceeds 2,097,152 words (only possible with a filter over more than 262,080 columns) the
 * call fails with DSX_EINVAL.  Results are those of dsx_topk_filtered / dsx_topk, bit for bit.  All calls on a GPU share the
 * one array: calls that overlap on one GPU (several lanes, several threads) race. */
int dsx_topk_filtered_static(const float* in, float* keys, uint32_t* values, uint32_t batch, uint32_t width, uint32_t k,
                             uint32_t position, const uint32_t* index, const uint64_t* filter_start, const uint64_t* filter_end,
                             const uint32_t* filter_index, const float* filter_mul);

/* Top-K (optionally filtered, as dsx_topk_filtered; filter_index == NULL: unfiltered, as dsx_topk) of a score matrix whose
 * producer left segment maxima (dsx_fc_forward_segmax): same results as the scanning calls, but only the segments that can
 * hold a result are read.  seg_max must describe `in` exactly (same batch rows, seg_width 64); with seg_max == NULL,
 * seg_width == 0, k > 64 or more than 2048 segments the call is the scanning one. */
int dsx_topk_guided(const float* in, float* keys, uint32_t* values, uint32_t batch, uint32_t width, uint32_t k, const float* seg_max,
                    uint32_t seg_width, uint32_t position, const uint32_t* index, const uint64_t* filter_start,
                    const uint64_t* filter_end, const uint32_t* filter_index, const float* filter_mul);

/* Output layer and recommendations in one call: the forward GEMM of NNLayer::ForwardPropagateFullyConnected (bias, product,
 * activation; engine/NNLayer.cpp:994-1167) on the output layer, followed by NNRecsGenerator::generateRecs' filtered
 * kCalculateTopK (utils/NNRecsGenerator.cpp:83-150) over its result, without ever storing the [batch x n] result:
 *   keys/values[b] = top-k over columns j of act(bias[j] + sum_i X[b][i] * W[i][j]), the scores of the columns listed in row b's
 * filter multiplied by 0 (filter arguments and semantics as dsx_topk_filtered with filter_mul == NULL: a listed column keeps
 * its place with a score of 0 and comes back when fewer than k scores lie above 0; filter_index == NULL: no filter).  W is [k_dim x n]
 * row-major.  Only the first few thousand columns are produced as a matrix (library scratch) and scanned; every later column
 * range is compared with the rows' running k-th scores inside the GEMM kernel's registers and only the survivors are kept.
 * Results are exact under the same total order as dsx_topk (score descending, column ascending); a score here and the same
 * score from dsx_fc_forward may differ in the last place (the bias enters the sum first instead of last).  A row whose
 * survivor list fills up (thousands of scores tied at the top), or whose k-th score is not above 0 while its filter lists columns
 * beyond the first block, is recomputed on the device, slowly; dsx_fc_topk_flagged tells
 * a caller that this has happened, so that it can go back to dsx_fc_forward + dsx_topk_filtered for such data.
 * Returns DSX_EUNSUPPORTED (dsx_fc_topk_supported() == 0) unless the activation is non-decreasing (sigmoid, tanh, ReLU, leaky
 * ReLU with a positive slope, linear) and X is 16-byte aligned with ldx a multiple of 4. */
int dsx_fc_topk(const float* X, uint32_t ldx, const float* W, const float* bias, uint32_t batch, uint32_t k_dim, uint32_t n,
                uint32_t activation, const dsx_act_params* params, uint32_t k, float* keys, uint32_t* values, uint32_t position,
                const uint32_t* index, const uint64_t* filter_start, const uint64_t* filter_end, const uint32_t* filter_index);
/* dsx_fc_topk with the products formed from bf16 matrix instructions (dsx_fc_forward_split): x_planes = dsx_fc_split of X,
 * w_planes = dsx_fc_split of W (k_major).  X and W are still needed: rows whose survivor lists fill up are recomputed from them. */
int dsx_fc_topk_split(const float* X, uint32_t ldx, const float* W, const void* x_planes, const void* w_planes, const float* bias,
                      uint32_t batch, uint32_t k_dim, uint32_t n, uint32_t activation, const dsx_act_params* params, uint32_t k, float* keys,
                      uint32_t* values, uint32_t position, const uint32_t* index, const uint64_t* filter_start, const uint64_t* filter_end,
                      const uint32_t* filter_index);
int dsx_fc_topk_supported(uint32_t ldx, const float* X, uint32_t activation, const dsx_act_params* params, const float* filter_mul);
/* 1 if any row of any dsx_fc_topk call so far had to be recomputed (reset != 0 clears the mark); dsx_fc_topk_flagged_for: the
 * same for the calls with this weight matrix only (the mark is kept per W pointer, for the 64 matrices used last). */
int dsx_fc_topk_flagged(int reset);
int dsx_fc_topk_flagged_for(const float* W, int reset);

/* ---- KNN ------------------------------------------------------------------------------------------------------------- */
/* Device part of KnnExactGpu::search (knn/KnnExactGpu.cu:99-148): scores = queries . items^T (cublasSgemmEx) followed by
 * the padded top-K.  items is column-major [rows_padded x dim] as KnnData::load builds it (knn/KnnData.cpp:197-207),
 * i.e. items[d * rows_padded + m]; queries is row-major [num_queries x dim]; the score matrix is produced in column
 * blocks inside the call and never stored whole: the first block goes through a scratch matrix and the scanning top-K,
 * later column ranges only append the scores that reach a query's running k-th score to candidate lists (exact; if a list
 * fills up the call notices at its end and repeats the search block by block).  The call returns when the results are
 * complete on the device.  workspace (device, 256-byte aligned, workspace_bytes) may be NULL: the library then
 * allocates what it needs for the call.  elapsed_ms (optional, 2 floats) receives the GEMM and top-K times like
 * KnnData::elapsedSgemm / elapsedTopK. */
int dsx_knn_search(const float* items, uint32_t rows_padded, uint32_t padding, uint32_t dim, const float* queries,
                   uint32_t num_queries, uint32_t k, float* scores, uint32_t* indexes, void* workspace, size_t workspace_bytes,
                   float* elapsed_ms);
size_t dsx_knn_workspace_bytes(uint32_t rows_padded, uint32_t dim, uint32_t num_queries, uint32_t k);
/* fp16 storage (astdl::knn::DataType::FP16).  The reference converts the column-major table once (KnnData::load,
 * knn/KnnData.cpp:209-216, kFloatToHalf of knn/MathUtil.cu:33-81: round to nearest even) and every query batch before the
 * GEMM (knn/KnnExactGpu.cu:108-116), multiplies fp16 operands and keeps fp32 scores.  Same arithmetic here; the fp16 table's
 * layout is this library's own: dsx_knn_f16_convert_items turns the fp32 column-major device table (as dsx_knn_search takes
 * it) into it, items_f16 (device, 16-byte aligned) holding dsx_knn_f16_table_bytes(rows_padded, dim) bytes; the fp32 table
 * can be freed afterwards.  dsx_knn_search_f16 takes fp32 queries like dsx_knn_search and converts them in its workspace. */
size_t dsx_knn_f16_table_bytes(uint32_t rows_padded, uint32_t dim);
int dsx_knn_f16_convert_items(const float* items, uint32_t rows_padded, uint32_t padding, uint32_t dim, void* items_f16);
int dsx_knn_search_f16(const void* items_f16, uint32_t rows_padded, uint32_t padding, uint32_t dim, const float* queries,
                       uint32_t num_queries, uint32_t k, float* scores, uint32_t* indexes, void* workspace, size_t workspace_bytes,
                       float* elapsed_ms);
size_t dsx_knn_workspace_bytes_f16(uint32_t rows_padded, uint32_t dim, uint32_t num_queries, uint32_t k);

/* dsx_knn_search with every fp32 product formed from bf16 matrix instructions (see dsx_fc_forward_split: as close to the exact
 * inner products as fp32 multiplication, not bit-identical to it; no counterpart in the reference).  item_planes: the table
 * as dsx_fc_split(items, rows_padded, 1, rows_padded, dim, item_planes) leaves it (dsx_fc_split_bytes(rows_padded, dim) bytes,
 * 1.5 x the table; made once, the fp32 table can be freed afterwards); queries are fp32 and split in the workspace, which
 * dsx_knn_workspace_bytes_split sizes.  Everything else as dsx_knn_search. */
int dsx_knn_search_split(const void* item_planes, uint32_t rows_padded, uint32_t padding, uint32_t dim, const float* queries,
                         uint32_t num_queries, uint32_t k, float* scores, uint32_t* indexes, void* workspace, size_t workspace_bytes,
                         float* elapsed_ms);
size_t dsx_knn_workspace_bytes_split(uint32_t rows_padded, uint32_t dim, uint32_t num_queries, uint32_t k);
/* No counterpart in the reference: how the last dsx_knn_search of this process ran. */
#define DSX_KNN_PATH_BLOCKS 0             /* every column block through the scratch score matrix and the scanning top-K */
#define DSX_KNN_PATH_CANDIDATES 1         /* first block as above, then candidate lists */
#define DSX_KNN_PATH_CANDIDATES_REDONE 2  /* a candidate list filled up: repeated block by block */
int dsx_knn_last_search_path(void);
/* dsx_knn_search_f16 scores the column ranges after the first block one workgroup per tile, or, when a range has enough item
 * tiles, with workgroups that keep their queries and walk a chunk of the range each (private candidate lists, no atomics on
 * device memory): the queries in registers when the vectors have at most 256 components, 128 queries per workgroup staged
 * through LDS otherwise.  The results are the same either way. */

#ifdef __cplusplus
}
#endif
#endif /* DSX_H */
