// dsx_runtime.hip — context, memory and timing entry points of libdsx_hip.so.
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>
#include "dsx_internal.h"

namespace dsx {

Context& ctx()
{
    static Context c;
    return c;
}

static thread_local char g_error[1024] = "";

int set_error(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

}  // namespace dsx
// How many launches DSX_SYNC=1 has waited for so far (a plain exported counter for the tests; not a function of the ABI).
extern "C" int dsx_debug_sync_launches;
int dsx_debug_sync_launches = 0;
namespace dsx {

int sync_after_launch(const char* fn, const char* kernel)
{
    hipStream_t s = ctx().stream;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return DSX_OK;
    }
    const hipError_t e = hipStreamSynchronize(s);
    if (e != hipSuccess) return set_error(DSX_EHIP, "%s: kernel %s failed: %s", fn, kernel, hipGetErrorString(e));
    ++dsx_debug_sync_launches;
    return DSX_OK;
}

static std::mutex g_alloc_mutex;
static std::map<void*, size_t> g_device_allocs;
static std::map<void*, size_t> g_host_allocs;

static std::vector<LibScratch*> g_lib_scratch;

int lib_scratch_reserve(LibScratch& s, size_t bytes, const char* what)
{
    if (bytes <= s.bytes) return DSX_OK;
    std::lock_guard<std::mutex> lock(g_alloc_mutex);
    if (s.ptr) {
        DSX_HIP(hipStreamSynchronize(ctx().stream));
        DSX_HIP(hipFree(s.ptr));
        ctx().gpu_bytes -= s.bytes;
        s.ptr = nullptr;
        s.bytes = 0;
    }
    hipError_t e = hipMalloc(&s.ptr, bytes);
    if (e != hipSuccess) {
        s.ptr = nullptr;
        return set_error(DSX_ENOMEM, "%s: cannot allocate %zu bytes: %s", what, bytes, hipGetErrorString(e));
    }
    s.bytes = bytes;
    ctx().gpu_bytes += bytes;
    if (!s.listed) {
        s.listed = true;
        g_lib_scratch.push_back(&s);
    }
    return DSX_OK;
}

static std::vector<void (*)()> g_shutdown_hooks;
void at_shutdown(void (*fn)())
{
    for (auto f : g_shutdown_hooks)
        if (f == fn) return;
    g_shutdown_hooks.push_back(fn);
}

static void lib_scratch_release()
{
    for (LibScratch* s : g_lib_scratch) {
        if (s->ptr) hipFree(s->ptr);
        s->ptr = nullptr;
        s->bytes = 0;
    }
}

}  // namespace dsx

using namespace dsx;

// Uploads of up to kUploadSlotBytes go through a ring of pinned staging buffers: the caller's bytes are copied into a slot,
// the DMA is queued on the selected lane's stream and the call returns — the source may be reused at once (as after the
// blocking cudaMemcpy of GpuBuffer::Upload), and everything queued later on the stream sees the data.  A batch's CSR arrays
// (four uploads, engine/NNTypes.cpp:583-778) then cost four host copies instead of four round trips.  Consecutive uploads
// share a slot until it is full (a batch of config 2 is 0.6 MB: the ring holds some fifty batches, so a caller that streams
// batches is never held up by the ring while the device is several batches behind); a slot is reused only after the copies
// out of it have finished on every lane.
constexpr int kUploadSlots = 8;
constexpr size_t kUploadSlotBytes = (size_t)4 << 20;
static char* g_upload_host[kUploadSlots] = {};
static hipEvent_t g_upload_done[kUploadSlots][DSX_MAX_LANES] = {};   // [slot][lane]: after the slot's last copy on that lane
static bool g_upload_busy[kUploadSlots][DSX_MAX_LANES] = {};    // an event has been recorded and not yet waited for
static bool g_upload_dirty[kUploadSlots][DSX_MAX_LANES] = {};   // copies queued since the slot was opened, no event recorded yet
static int g_upload_slot = 0;       // slot being filled
static size_t g_upload_fill = 0;    // bytes of it handed out

// Downloads of up to kUploadSlotBytes land in a pinned buffer first and are copied to the caller's memory by the host: a copy
// straight into pageable memory costs the runtime a staging round trip of its own that is several times slower.
static char* g_download_host = nullptr;

static int download_small(void* dst, const void* src, size_t bytes, hipStream_t s, size_t slot_offset)
{
    if (!g_download_host) DSX_HIP(hipHostMalloc((void**)&g_download_host, kUploadSlotBytes, hipHostMallocDefault));
    DSX_HIP(hipMemcpyAsync(g_download_host + slot_offset, src, bytes, hipMemcpyDeviceToHost, s));
    (void)dst;
    return DSX_OK;
}

static void upload_ring_release()
{
    if (g_download_host) hipHostFree(g_download_host);
    g_download_host = nullptr;
    for (int i = 0; i < kUploadSlots; i++) {
        if (g_upload_host[i]) hipHostFree(g_upload_host[i]);
        g_upload_host[i] = nullptr;
        for (int l = 0; l < DSX_MAX_LANES; l++) {
            if (g_upload_done[i][l]) hipEventDestroy(g_upload_done[i][l]);
            g_upload_done[i][l] = nullptr;
            g_upload_busy[i][l] = false;
            g_upload_dirty[i][l] = false;
        }
    }
    g_upload_slot = 0;
    g_upload_fill = 0;
}


// Lanes: up to DSX_MAX_LANES independent in-order streams, so that the kernels of several batches can be in flight together
// (one batch's top-K and input layers fill the gaps of another's GEMM).  ctx().stream is always the selected lane's stream;
// everything the library launches goes there.  Operations whose effect every lane must see in order — uploads, clears,
// device copies, allocation fills, timers — join the lanes around themselves; downloads and dsx_sync wait for all of them.
// A lane's stream is made when the lane is first selected; lane 0 is the context's own stream.
static hipStream_t g_lane_stream[DSX_MAX_LANES] = {};
static hipEvent_t g_lane_event[DSX_MAX_LANES] = {};   // [l]: last join point recorded on lane l
static int g_lane = 0;

namespace dsx {
int current_lane() { return g_lane; }
}  // namespace dsx

static bool lanes_in_use() { return g_lane_stream[0] != nullptr; }

// Work can only be queued on a lane while it is selected, so "lane o has been selected since lane l last waited for it" is
// all that has to be tracked: a burst of uploads between two batches then costs one cross-stream wait per lane, not one per
// call (each is an event record, a wait and a barrier packet between two hardware queues).
static uint32_t g_lane_selected[DSX_MAX_LANES] = {1, 0};                 // how often each lane has been selected
static uint32_t g_lane_seen[DSX_MAX_LANES][DSX_MAX_LANES] = {};         // [l][o]: g_lane_selected[o] when lane l last waited for lane o
static bool g_lane_publish[DSX_MAX_LANES][DSX_MAX_LANES] = {};          // [l][o]: lane l holds ordered work lane o has not been told to wait for

// Lane `waiter` waits for everything queued so far on lane o.
static int lane_wait_for(int waiter, int o)
{
    DSX_HIP(hipEventRecord(g_lane_event[o], g_lane_stream[o]));
    DSX_HIP(hipStreamWaitEvent(g_lane_stream[waiter], g_lane_event[o], 0));
    g_lane_seen[waiter][o] = g_lane_selected[o];
    g_lane_publish[o][waiter] = false;
    return DSX_OK;
}

// The selected lane waits for everything queued so far on the other ones.
static int lanes_join_before()
{
    if (!lanes_in_use()) return DSX_OK;
    for (int o = 0; o < DSX_MAX_LANES; o++) {
        if (o == g_lane || !g_lane_stream[o]) continue;
        if (g_lane_seen[g_lane][o] != g_lane_selected[o] || g_lane_publish[o][g_lane])
            if (int rc = lane_wait_for(g_lane, o)) return rc;
    }
    return DSX_OK;
}

// The other lanes must wait for what was just queued on the selected one: arranged when one of them is selected next.
static int lanes_join_after()
{
    if (!lanes_in_use()) return DSX_OK;
    for (int o = 0; o < DSX_MAX_LANES; o++)
        if (o != g_lane) g_lane_publish[g_lane][o] = true;   // (also for lanes that do not exist yet: they start after everything anyway)
    return DSX_OK;
}

static void lanes_release()
{
    // lane 0's stream is ctx().stream's original and is destroyed with the context
    for (int l = 1; l < DSX_MAX_LANES; l++)
        if (g_lane_stream[l]) hipStreamDestroy(g_lane_stream[l]);
    for (auto& e : g_lane_event)
        if (e) hipEventDestroy(e);
    for (int l = 0; l < DSX_MAX_LANES; l++) {
        g_lane_stream[l] = nullptr;
        g_lane_event[l] = nullptr;
        g_lane_selected[l] = (l == 0) ? 1 : 0;
        for (int o = 0; o < DSX_MAX_LANES; o++) {
            g_lane_seen[l][o] = 0;
            g_lane_publish[l][o] = false;
        }
    }
    g_lane = 0;
}

// Holds a workgroup's place (registers, a slot of every SIMD) without issuing vector or memory instructions.
template <int REGS>
__global__ __launch_bounds__(256) void occupy_kernel(uint32_t cycles)
{
    if (REGS == 128) asm volatile("v_mov_b32 v127, 0" ::: "v127");   // the highest register named fixes the allocation
    if (REGS == 64) asm volatile("v_mov_b32 v63, 0" ::: "v63");
    const uint64_t t0 = __builtin_readcyclecounter();
    for (uint32_t spins = 0; spins < 100000 && __builtin_readcyclecounter() - t0 < cycles; spins++) __builtin_amdgcn_s_sleep(8);
}

extern "C" {

const char* dsx_last_error(void) { return g_error; }

int dsx_is_initialized(void) { return ctx().initialized ? 1 : 0; }

int dsx_init(int device)
{
    Context& c = ctx();
    if (c.initialized) {
        if (c.device == device) {
            ++c.users;   // every dsx_init is paired with a dsx_shutdown; the last one tears the context down
            return DSX_OK;
        }
        return set_error(DSX_EINVAL, "dsx_init: already initialised on device %d (one context per process)", c.device);
    }
    int count = 0;
    DSX_HIP(hipGetDeviceCount(&count));
    if (count < 1) return set_error(DSX_EHIP, "dsx_init: no HIP device is visible");
    DSX_CHECK_ARG(device >= 0 && device < count, "dsx_init: device %d out of range (%d visible)", device, count);
    DSX_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    DSX_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return set_error(DSX_EUNSUPPORTED, "dsx_init: device %d is %s; this library is built for gfx950 only", device, prop.gcnArchName);
    if (int rc = topk_static_setup(device)) return rc;
    DSX_HIP(hipStreamCreateWithFlags(&c.stream, hipStreamNonBlocking));
    DSX_HIP(hipEventCreate(&c.ev_start));
    DSX_HIP(hipEventCreate(&c.ev_stop));
    c.device = device;
    c.num_cus = prop.multiProcessorCount;
    c.initialized = true;
    c.users = 1;
    const char* sync = getenv("DSX_SYNC");
    c.sync_launches = sync && sync[0] != '\0' && strcmp(sync, "0") != 0;
    return DSX_OK;
}

int dsx_shutdown(void)
{
    Context& c = ctx();
    if (!c.initialized) return DSX_OK;
    if (--c.users > 0) return DSX_OK;
    for (int l = 1; l < DSX_MAX_LANES; l++)
        if (g_lane_stream[l]) hipStreamSynchronize(g_lane_stream[l]);
    if (g_lane_stream[0]) c.stream = g_lane_stream[0];
    hipStreamSynchronize(c.stream);
    for (auto fn : g_shutdown_hooks) fn();
    g_shutdown_hooks.clear();
    lanes_release();
    upload_ring_release();
    {
        std::lock_guard<std::mutex> lock(g_alloc_mutex);
        lib_scratch_release();
        for (auto& kv : g_device_allocs) hipFree(kv.first);
        for (auto& kv : g_host_allocs) hipHostFree(kv.first);
        g_device_allocs.clear();
        g_host_allocs.clear();
        c.gpu_bytes = c.cpu_bytes = 0;
    }
    hipEventDestroy(c.ev_start);
    hipEventDestroy(c.ev_stop);
    hipStreamDestroy(c.stream);
    c = Context();
    return DSX_OK;
}

int dsx_testing_occupy(uint32_t workgroups, uint32_t cycles, uint32_t vgprs)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(workgroups >= 1 && workgroups <= 65536 && cycles <= 10000000u, "dsx_testing_occupy: %u workgroups, %u cycles", workgroups, cycles);
    hipStream_t s = ctx().stream;
    if (vgprs == 128) hipLaunchKernelGGL((occupy_kernel<128>), dim3(workgroups), dim3(256), 0, s, cycles);
    else if (vgprs == 64) hipLaunchKernelGGL((occupy_kernel<64>), dim3(workgroups), dim3(256), 0, s, cycles);
    else hipLaunchKernelGGL((occupy_kernel<0>), dim3(workgroups), dim3(256), 0, s, cycles);
    DSX_LAUNCH_CHECK("occupy_kernel");
    return DSX_OK;
}

int dsx_testing_reset(void)
{
    ctx().knobs = TestKnobs();
    return DSX_OK;
}

int dsx_get_device_info(dsx_device_info* info)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(info, "dsx_get_device_info: null info");
    hipDeviceProp_t prop;
    DSX_HIP(hipGetDeviceProperties(&prop, ctx().device));
    memset(info, 0, sizeof(*info));
    strncpy(info->name, prop.name, sizeof(info->name) - 1);
    strncpy(info->arch, prop.gcnArchName, sizeof(info->arch) - 1);
    info->compute_units = prop.multiProcessorCount;
    info->wavefront_size = prop.warpSize;
    info->lds_bytes_per_cu = (int)prop.sharedMemPerBlock;
    info->hbm_bytes = prop.totalGlobalMem;
    size_t free_b = 0, total_b = 0;
    DSX_HIP(hipMemGetInfo(&free_b, &total_b));
    info->hbm_free_bytes = free_b;
    info->clock_khz = prop.clockRate;
    info->memory_clock_khz = prop.memoryClockRate;
    return DSX_OK;
}

int dsx_get_memory_usage(int* gpu_kib, int* cpu_kib)
{
    if (gpu_kib) *gpu_kib = (int)(ctx().gpu_bytes / 1024);
    if (cpu_kib) *cpu_kib = (int)(ctx().cpu_bytes / 1024);
    return DSX_OK;
}

void* dsx_stream(void) { return (void*)ctx().stream; }

int dsx_set_lane(int lane)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(lane >= 0 && lane < DSX_MAX_LANES, "dsx_set_lane: lane %d (0..%d)", lane, DSX_MAX_LANES - 1);
    if (!lanes_in_use()) {
        if (lane == 0) return DSX_OK;   // nothing to set up until another lane is asked for
        g_lane_stream[0] = ctx().stream;
        DSX_HIP(hipEventCreateWithFlags(&g_lane_event[0], hipEventDisableTiming));
    }
    if (!g_lane_stream[lane]) {
        DSX_HIP(hipStreamCreateWithFlags(&g_lane_stream[lane], hipStreamNonBlocking));
        DSX_HIP(hipEventCreateWithFlags(&g_lane_event[lane], hipEventDisableTiming));
        // the new lane starts after everything queued so far on the others
        for (int o = 0; o < DSX_MAX_LANES; o++)
            if (o != lane && g_lane_stream[o])
                if (int rc = lane_wait_for(lane, o)) return rc;
    }
    if (lane != g_lane) {
        // ordered work (uploads, clears, copies) of the lanes that published some: the new lane runs after it
        for (int o = 0; o < DSX_MAX_LANES; o++)
            if (o != lane && g_lane_stream[o] && g_lane_publish[o][lane])
                if (int rc = lane_wait_for(lane, o)) return rc;
        g_lane = lane;
        g_lane_selected[lane]++;
        ctx().stream = g_lane_stream[lane];
    }
    return DSX_OK;
}

int dsx_get_lane(void) { return g_lane; }

int dsx_malloc(void** p, size_t bytes)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(p, "dsx_malloc: null result pointer");
    *p = nullptr;
    if (bytes == 0) bytes = 4;
    hipError_t e = hipMalloc(p, bytes);
    if (e != hipSuccess) return set_error(DSX_ENOMEM, "dsx_malloc: hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    DSX_HIP(hipMemsetAsync(*p, 0, bytes, ctx().stream));
    if (int rc = lanes_join_after()) return rc;
    std::lock_guard<std::mutex> lock(g_alloc_mutex);
    g_device_allocs[*p] = bytes;
    ctx().gpu_bytes += bytes;
    return DSX_OK;
}

int dsx_malloc_managed(void** p, size_t bytes)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(p, "dsx_malloc_managed: null result pointer");
    *p = nullptr;
    if (bytes == 0) bytes = 4;
    // Fine-grained pinned host memory mapped into the device: host-dereferenceable without page migration.
    hipError_t e = hipHostMalloc(p, bytes, hipHostMallocMapped | hipHostMallocPortable);
    if (e != hipSuccess) return set_error(DSX_ENOMEM, "dsx_malloc_managed: hipHostMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    memset(*p, 0, bytes);
    std::lock_guard<std::mutex> lock(g_alloc_mutex);
    g_host_allocs[*p] = bytes;
    ctx().cpu_bytes += bytes;
    return DSX_OK;
}

int dsx_malloc_host(void** p, size_t bytes)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(p, "dsx_malloc_host: null result pointer");
    *p = nullptr;
    if (bytes == 0) bytes = 4;
    hipError_t e = hipHostMalloc(p, bytes, hipHostMallocDefault);
    if (e != hipSuccess) return set_error(DSX_ENOMEM, "dsx_malloc_host: hipHostMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    std::lock_guard<std::mutex> lock(g_alloc_mutex);
    g_host_allocs[*p] = bytes;
    ctx().cpu_bytes += bytes;
    return DSX_OK;
}

int dsx_free(void* p)
{
    if (!p) return DSX_OK;
    DSX_REQUIRE_INIT();
    {
        std::lock_guard<std::mutex> lock(g_alloc_mutex);
        auto it = g_device_allocs.find(p);
        if (it == g_device_allocs.end()) {
            auto ih = g_host_allocs.find(p);
            if (ih == g_host_allocs.end()) return set_error(DSX_EINVAL, "dsx_free: %p was not allocated by this library", p);
            ctx().cpu_bytes -= ih->second;
            g_host_allocs.erase(ih);
            DSX_HIP(hipStreamSynchronize(ctx().stream));
            DSX_HIP(hipHostFree(p));
            return DSX_OK;
        }
        ctx().gpu_bytes -= it->second;
        g_device_allocs.erase(it);
    }
    DSX_HIP(hipStreamSynchronize(ctx().stream));
    DSX_HIP(hipFree(p));
    return DSX_OK;
}

int dsx_free_host(void* p) { return dsx_free(p); }

int dsx_memset(void* p, int value, size_t bytes)
{
    DSX_REQUIRE_INIT();
    if (bytes == 0) return DSX_OK;
    DSX_CHECK_ARG(p, "dsx_memset: null pointer");
    if (int rc = lanes_join_before()) return rc;
    DSX_HIP(hipMemsetAsync(p, value, bytes, ctx().stream));
    return lanes_join_after();
}

// Copies up to four arrays from pinned host memory to device memory, 16 bytes per lane and step.  Destinations and sources
// are 16-byte aligned.
constexpr int kUploadPieces = 4;
struct UploadPieces {
    char* dst[kUploadPieces];
    const char* src[kUploadPieces];
    uint32_t bytes[kUploadPieces];
};

__global__ __launch_bounds__(256) void upload_pieces_kernel(UploadPieces p)
{
#pragma unroll
    for (int i = 0; i < kUploadPieces; i++) {
        const uint32_t units = p.bytes[i] / 16;
        for (uint32_t u = blockIdx.x * 256 + threadIdx.x; u < units; u += gridDim.x * 256)
            reinterpret_cast<uint4*>(p.dst[i])[u] = reinterpret_cast<const uint4*>(p.src[i])[u];
        if (blockIdx.x == 0) {
            const uint32_t t = units * 16 + threadIdx.x;
            if (t < p.bytes[i]) p.dst[i][t] = p.src[i][t];
        }
    }
}

// Makes room for `bytes` in the ring (all in one slot) and returns where; moves on to the next slot when the current one
// is full, once nothing is being copied out of that one any more.  g_alloc_mutex is held.
static int upload_ring_take(size_t bytes, char** staged, int* slot_out)
{
    if (g_upload_fill + bytes > kUploadSlotBytes) {
        // The slot that is full: one event per lane that copied out of it, recorded now — behind its last copy on that lane's
        // in-order stream, if later than strictly needed — instead of one behind every upload.
        for (int l = 0; l < DSX_MAX_LANES; l++)
            if (g_upload_dirty[g_upload_slot][l]) {
                DSX_HIP(hipEventRecord(g_upload_done[g_upload_slot][l], g_lane_stream[l] ? g_lane_stream[l] : ctx().stream));
                g_upload_dirty[g_upload_slot][l] = false;
                g_upload_busy[g_upload_slot][l] = true;
            }
        g_upload_slot = (g_upload_slot + 1) % kUploadSlots;
        g_upload_fill = 0;
        for (int l = 0; l < DSX_MAX_LANES; l++)
            if (g_upload_busy[g_upload_slot][l]) {
                DSX_HIP(hipEventSynchronize(g_upload_done[g_upload_slot][l]));
                g_upload_busy[g_upload_slot][l] = false;
            }
    }
    const int slot = g_upload_slot;
    if (!g_upload_host[slot]) {
        DSX_HIP(hipHostMalloc((void**)&g_upload_host[slot], kUploadSlotBytes, hipHostMallocDefault));
        for (int l = 0; l < DSX_MAX_LANES; l++) DSX_HIP(hipEventCreateWithFlags(&g_upload_done[slot][l], hipEventDisableTiming));
    }
    *staged = g_upload_host[slot] + g_upload_fill;
    *slot_out = slot;
    g_upload_fill += (bytes + 255) / 256 * 256;
    return DSX_OK;
}

// Host memory -> device on the selected lane's stream, several arrays at once.  What fits the pinned ring is staged there and
// copied by upload_pieces_kernel, which reads the staging memory over the bus itself, four arrays to a launch (three
// copy-engine transfers for a batch's CSR arrays of 0.4 MB: 50 us until the device has them; one launch: 33.  A launch per
// 128 KiB, so that the host stages a piece while the device copies the one before, costs more in launches than it hides).
// The call returns when everything is queued; the sources may be reused at once.  An array that does not fit the ring,
// or whose destination is not 16-byte aligned, is copied by the copy engine (the large one straight from the caller's
// memory, which may be pageable, and waited for).
static int upload_on_selected_lane(int count, void* const* dst, const void* const* src, const size_t* bytes)
{
    std::lock_guard<std::mutex> lock(g_alloc_mutex);
    UploadPieces p{};
    int held = 0;
    size_t held_bytes = 0;
    auto launch = [&]() -> int {
        if (held == 0) return DSX_OK;
        for (int i = held; i < kUploadPieces; i++) p.bytes[i] = 0;
        const unsigned blocks = (unsigned)std::min<size_t>((held_bytes / 16 + 255) / 256 + 1, 2048);
        hipLaunchKernelGGL(upload_pieces_kernel, dim3(blocks), dim3(256), 0, ctx().stream, p);
        DSX_LAUNCH_CHECK("upload_pieces_kernel");
        held = 0;
        held_bytes = 0;
        return DSX_OK;
    };
    for (int a = 0; a < count; a++) {
        if (bytes[a] == 0) continue;
        if (bytes[a] > kUploadSlotBytes) {
            if (int rc = launch()) return rc;
            DSX_HIP(hipMemcpyAsync(dst[a], src[a], bytes[a], hipMemcpyHostToDevice, ctx().stream));
            DSX_HIP(hipStreamSynchronize(ctx().stream));   // src may be pageable: wait until it has been read
            continue;
        }
        char* staged = nullptr;
        int slot = 0;
        if (g_upload_fill + bytes[a] > kUploadSlotBytes)   // the ring moves on: what reads the full slot is queued before its event
            if (int rc = launch()) return rc;
        if (int rc = upload_ring_take(bytes[a], &staged, &slot)) return rc;
        g_upload_dirty[slot][g_lane] = true;
        if (((uintptr_t)dst[a] & 15) != 0) {
            memcpy(staged, src[a], bytes[a]);
            DSX_HIP(hipMemcpyAsync(dst[a], staged, bytes[a], hipMemcpyHostToDevice, ctx().stream));
            continue;
        }
        memcpy(staged, src[a], bytes[a]);
        p.dst[held] = (char*)dst[a];
        p.src[held] = staged;
        p.bytes[held] = (uint32_t)bytes[a];
        held++;
        held_bytes += bytes[a];
        if (held == kUploadPieces)
            if (int rc = launch()) return rc;
    }
    return launch();
}

static int upload_on_selected_lane(void* dst, const void* src, size_t bytes)
{
    return upload_on_selected_lane(1, &dst, &src, &bytes);
}

int dsx_memcpy_h2d(void* dst, const void* src, size_t bytes)
{
    DSX_REQUIRE_INIT();
    if (bytes == 0) return DSX_OK;
    DSX_CHECK_ARG(dst && src, "dsx_memcpy_h2d: null pointer");
    // the destination may still be read by kernels of another lane, and is read by whatever any lane runs next
    if (int rc = lanes_join_before()) return rc;
    if (int rc = upload_on_selected_lane(dst, src, bytes)) return rc;
    return lanes_join_after();
}

int dsx_memcpy_h2d_unordered(void* dst, const void* src, size_t bytes)
{
    DSX_REQUIRE_INIT();
    if (bytes == 0) return DSX_OK;
    DSX_CHECK_ARG(dst && src, "dsx_memcpy_h2d_unordered: null pointer");
    return upload_on_selected_lane(dst, src, bytes);
}

int dsx_memcpy_h2d_unordered_many(int count, void* const* dst, const void* const* src, const size_t* bytes)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(count >= 0 && (count == 0 || (dst && src && bytes)), "dsx_memcpy_h2d_unordered_many: null argument");
    for (int a = 0; a < count; a++) DSX_CHECK_ARG(bytes[a] == 0 || (dst[a] && src[a]), "dsx_memcpy_h2d_unordered_many: null pointer (array %d)", a);
    return upload_on_selected_lane(count, dst, src, bytes);
}

int dsx_lane_wait_other(void)
{
    DSX_REQUIRE_INIT();
    if (!lanes_in_use()) return DSX_OK;
    for (int o = 0; o < DSX_MAX_LANES; o++)
        if (o != g_lane && g_lane_stream[o])
            if (int rc = lane_wait_for(g_lane, o)) return rc;
    return DSX_OK;
}

// Host-side wait for every lane but the selected one.
static int sync_other_lanes()
{
    for (int o = 0; o < DSX_MAX_LANES; o++)
        if (o != g_lane && g_lane_stream[o]) DSX_HIP(hipStreamSynchronize(g_lane_stream[o]));
    return DSX_OK;
}

int dsx_memcpy_d2h(void* dst, const void* src, size_t bytes)
{
    DSX_REQUIRE_INIT();
    if (bytes == 0) return DSX_OK;
    DSX_CHECK_ARG(dst && src, "dsx_memcpy_d2h: null pointer");
    if (int rc = sync_other_lanes()) return rc;   // the data may come from any lane
    if (bytes <= kUploadSlotBytes) {
        std::lock_guard<std::mutex> lock(g_alloc_mutex);
        if (int rc = download_small(dst, src, bytes, ctx().stream, 0)) return rc;
        DSX_HIP(hipStreamSynchronize(ctx().stream));
        memcpy(dst, g_download_host, bytes);
        return DSX_OK;
    }
    DSX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx().stream));
    DSX_HIP(hipStreamSynchronize(ctx().stream));
    return DSX_OK;
}

// Two downloads with one wait (a top-K's scores and indexes): the second copy does not pay a round trip of its own.
int dsx_memcpy_d2h_pair(void* dst0, const void* src0, size_t bytes0, void* dst1, const void* src1, size_t bytes1)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG((bytes0 == 0 || (dst0 && src0)) && (bytes1 == 0 || (dst1 && src1)), "dsx_memcpy_d2h_pair: null pointer");
    if (int rc = sync_other_lanes()) return rc;   // the data may come from any lane
    const size_t off1 = (bytes0 + 255) / 256 * 256;
    if (off1 + bytes1 <= kUploadSlotBytes) {
        std::lock_guard<std::mutex> lock(g_alloc_mutex);
        if (bytes0) if (int rc = download_small(dst0, src0, bytes0, ctx().stream, 0)) return rc;
        if (bytes1) if (int rc = download_small(dst1, src1, bytes1, ctx().stream, off1)) return rc;
        DSX_HIP(hipStreamSynchronize(ctx().stream));
        if (bytes0) memcpy(dst0, g_download_host, bytes0);
        if (bytes1) memcpy(dst1, g_download_host + off1, bytes1);
        return DSX_OK;
    }
    if (bytes0) DSX_HIP(hipMemcpyAsync(dst0, src0, bytes0, hipMemcpyDeviceToHost, ctx().stream));
    if (bytes1) DSX_HIP(hipMemcpyAsync(dst1, src1, bytes1, hipMemcpyDeviceToHost, ctx().stream));
    DSX_HIP(hipStreamSynchronize(ctx().stream));
    return DSX_OK;
}

int dsx_memcpy_d2d(void* dst, const void* src, size_t bytes)
{
    DSX_REQUIRE_INIT();
    if (bytes == 0) return DSX_OK;
    DSX_CHECK_ARG(dst && src, "dsx_memcpy_d2d: null pointer");
    if (int rc = lanes_join_before()) return rc;
    DSX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx().stream));
    return lanes_join_after();
}

int dsx_sync(void)
{
    DSX_REQUIRE_INIT();
    if (int rc = sync_other_lanes()) return rc;
    DSX_HIP(hipStreamSynchronize(ctx().stream));
    return DSX_OK;
}

int dsx_sync_lane(int lane)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(lane >= 0 && lane < DSX_MAX_LANES, "dsx_sync_lane: lane %d (0..%d)", lane, DSX_MAX_LANES - 1);
    hipStream_t s = g_lane_stream[lane] ? g_lane_stream[lane] : ctx().stream;
    DSX_HIP(hipStreamSynchronize(s));
    return DSX_OK;
}

// Downloads that wait for one lane only: a caller that keeps two batches in flight reads one batch's results while the
// other batch runs.
int dsx_memcpy_d2h_lane(int lane, void* dst, const void* src, size_t bytes)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(lane >= 0 && lane < DSX_MAX_LANES, "dsx_memcpy_d2h_lane: lane %d (0..%d)", lane, DSX_MAX_LANES - 1);
    if (bytes == 0) return DSX_OK;
    DSX_CHECK_ARG(dst && src, "dsx_memcpy_d2h_lane: null pointer");
    hipStream_t s = g_lane_stream[lane] ? g_lane_stream[lane] : ctx().stream;
    if (bytes <= kUploadSlotBytes) {
        std::lock_guard<std::mutex> lock(g_alloc_mutex);
        if (int rc = download_small(dst, src, bytes, s, 0)) return rc;
        DSX_HIP(hipStreamSynchronize(s));
        memcpy(dst, g_download_host, bytes);
        return DSX_OK;
    }
    DSX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, s));
    DSX_HIP(hipStreamSynchronize(s));
    return DSX_OK;
}

int dsx_marker_create(void** marker)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(marker, "dsx_marker_create: null pointer");
    hipEvent_t e;
    DSX_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    *marker = (void*)e;
    return DSX_OK;
}

int dsx_marker_record(void* marker)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(marker, "dsx_marker_record: null marker");
    DSX_HIP(hipEventRecord((hipEvent_t)marker, ctx().stream));
    return DSX_OK;
}

int dsx_marker_wait(void* marker)
{
    DSX_REQUIRE_INIT();
    DSX_CHECK_ARG(marker, "dsx_marker_wait: null marker");
    DSX_HIP(hipEventSynchronize((hipEvent_t)marker));
    return DSX_OK;
}

int dsx_marker_destroy(void* marker)
{
    if (!marker) return DSX_OK;
    DSX_REQUIRE_INIT();
    DSX_HIP(hipEventDestroy((hipEvent_t)marker));
    return DSX_OK;
}

int dsx_timer_start(void)
{
    DSX_REQUIRE_INIT();
    if (int rc = lanes_join_before()) return rc;
    DSX_HIP(hipEventRecord(ctx().ev_start, ctx().stream));
    return lanes_join_after();
}

int dsx_timer_stop(float* elapsed_ms)
{
    DSX_REQUIRE_INIT();
    if (int rc = lanes_join_before()) return rc;
    DSX_HIP(hipEventRecord(ctx().ev_stop, ctx().stream));
    DSX_HIP(hipEventSynchronize(ctx().ev_stop));
    float ms = 0.0f;
    DSX_HIP(hipEventElapsedTime(&ms, ctx().ev_start, ctx().ev_stop));
    if (elapsed_ms) *elapsed_ms = ms;
    return DSX_OK;
}

}  // extern "C"
