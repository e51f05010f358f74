// Device, memory, stream and error plumbing of libtensor_hip — the part of the C ABI the reference obtains from the
// CUDA driver through ManagedCuda (Tensor/Tensor/Cuda/CudaUtils.fs:36-60 context, Cuda/CudaBackend.fs:54-93 storage,
// :206-270 transfers, Cuda/CudaRegMem.fs pinned memory, Cuda/CudaCfg.fs:16-27 stream).
#include "common.h"

#include <atomic>
#include <map>
#include <mutex>
#include <thread>
#include <vector>
#include <cctype>
#include <cstdlib>
#include <cstring>
#include <unordered_map>

namespace dnh {

namespace {
std::mutex g_mu;
std::atomic<uint64_t> g_epoch{1};   // bumped when the device is chosen
bool g_init = false;
int g_device = 0;
std::mutex g_pinned_mu;
std::map<uintptr_t, size_t> g_pinned;   // blocks handed out by dnh_host_alloc
int g_cus = 256;
std::map<hipStream_t, int32_t*> g_error_flags;   // one index-error word per stream, so concurrent streams do not see each other's errors

struct Workspace {
    std::mutex in_use;   // held through a WorkspaceLease while an entry point queues the kernels that use the buffer
    void* ptr = nullptr;
    size_t bytes = 0;
    // words through which the workgroups of one launch meet (arrival counters, tile descriptors): zero when allocated,
    // never used for anything else, so a kernel may rely on what the previous launch left there
    void* sync_ptr = nullptr;
    size_t sync_bytes = 0;
    uint32_t epoch = 0;   // counts the launches that used the words; 30 bits, the words are cleared when it wraps
};
std::map<hipStream_t, Workspace> g_ws;

// Stream-ordered block cache behind dnh_alloc_async / dnh_free_async.  A block released on stream S goes to S's free
// list and may be handed out again only to an allocation on S: work already queued on S that still touches the block
// runs before anything the new owner queues on S, so no wait is needed.  hipMalloc / hipFree (which synchronise the
// device) are left for cache misses, trimming and out-of-memory retries.
struct Pool {
    std::mutex mu;
    std::map<hipStream_t, std::multimap<size_t, void*>> free_blocks;
    std::unordered_map<void*, size_t> live;  // blocks handed out and not yet released -> rounded size
    size_t cached_bytes = 0, live_bytes = 0, limit_bytes = 0;  // limit 0 = keep everything until trimmed
    uint64_t hits = 0, misses = 0;
};
Pool g_pool;

size_t pool_round(size_t bytes) {
    if (bytes == 0) bytes = 1;
    const size_t g = bytes < ((size_t)1 << 20) ? 512 : ((size_t)2 << 20);
    return (bytes + g - 1) / g * g;
}

std::mutex g_dead_mu;
std::vector<hipStream_t> g_dead_streams;   // handles destroyed by dnh_stream_destroy (a later dnh_stream_create may get one again)

// caller holds g_pool.mu
int32_t pool_trim_locked() {
    if (g_pool.cached_bytes == 0) return DNH_OK;
    DNH_HIP(hipDeviceSynchronize());
    for (auto& per_stream : g_pool.free_blocks)
        for (auto& blk : per_stream.second) (void)hipFree(blk.second);
    g_pool.free_blocks.clear();
    g_pool.cached_bytes = 0;
    return DNH_OK;
}
// hipMalloc that gives the block cache back to the driver and tries once more when the driver is out of memory (the cache is
// unbounded by default and may hold most of the device's memory).  Caller does not hold g_pool.mu.
int32_t device_malloc(void** out, size_t bytes, const char* what) {
    hipError_t e = hipMalloc(out, bytes);
    if (e == hipErrorOutOfMemory) {
        (void)hipGetLastError();
        {
            std::lock_guard<std::mutex> lock(g_pool.mu);
            DNH_TRY(pool_trim_locked());
        }
        e = hipMalloc(out, bytes);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        *out = nullptr;
        if (e == hipErrorOutOfMemory) return fail(DNH_ERR_OUT_OF_MEMORY, "%s: device memory allocation of %zu MB failed", what, bytes >> 20);
        return fail(DNH_ERR_HIP, "%s: hipMalloc(%zu): %s", what, bytes, hipGetErrorString(e));
    }
    return DNH_OK;
}
}  // namespace

std::string& last_error() {
    thread_local std::string e;
    return e;
}

static int32_t init_locked(int device) {
    if (g_init && device == g_device) return DNH_OK;
    if (g_init) return fail(DNH_ERR_INVALID_ARG, "dnh_init: the library already runs on device %d; it cannot move to device %d", g_device, device);
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0) return fail(DNH_ERR_HIP, "no HIP device available (%s)", hipGetErrorString(e));
    if (device < 0 || device >= count) return fail(DNH_ERR_INVALID_ARG, "device %d out of range (0..%d)", device, count - 1);
    DNH_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    DNH_HIP(hipGetDeviceProperties(&prop, device));
    g_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    g_device = device;
    g_init = true;
    g_epoch.fetch_add(1, std::memory_order_release);
    return DNH_OK;
}

int32_t ensure_init() {
    // HIP's current device is per host thread: the first call of a thread binds the thread to the library's device; later
    // calls cost one thread-local compare.
    thread_local int t_bound_device = -1;
    thread_local uint64_t t_bound_epoch = 0;
    if (t_bound_device >= 0 && t_bound_epoch == g_epoch.load(std::memory_order_acquire)) return DNH_OK;
    std::lock_guard<std::mutex> lock(g_mu);
    if (!g_init) DNH_TRY(init_locked(0));
    DNH_HIP(hipSetDevice(g_device));
    t_bound_device = g_device;
    t_bound_epoch = g_epoch.load(std::memory_order_acquire);
    return DNH_OK;
}

int device_cus() { return g_cus; }

namespace {
struct OptionDef {
    const char* name;
    int def, lo, hi;
};
// order of enum Option
constexpr OptionDef kOptions[OPT_COUNT] = {
    {"dot_bf16x3", 1, 0, 1},       {"dot_f64_pinned", 1, 0, 1},    {"dot_big", -1, -1, 1},          {"dot_splits", 0, 0, 1 << 20},
    {"dot_int_mfma", 1, 0, 1},     {"tr4", 1, 0, 1},               {"scatter_fp_atomic", 0, 0, 1},  {"compact_one_pass", 0, 0, 1},
    {"count_one_launch", 1, 0, 1},
    {"lookback_spins", 1 << 18, 0, 1 << 30},
    {"invert_tournament", -1, -1, 1},
};
std::atomic<int> g_options[OPT_COUNT];
std::once_flag g_options_once;
void init_options() {
    std::call_once(g_options_once, [] {
        for (int o = 0; o < OPT_COUNT; o++) {
            std::string env = "DNH_";
            for (const char* c = kOptions[o].name; *c; c++) env += (char)toupper((unsigned char)*c);
            const char* e = getenv(env.c_str());
            int v = kOptions[o].def;
            if (e && *e) {
                v = atoi(e);
                if (v < kOptions[o].lo) v = kOptions[o].lo;
                if (v > kOptions[o].hi) v = kOptions[o].hi;
            }
            g_options[o].store(v, std::memory_order_relaxed);
        }
    });
}
int find_option(const char* name) {
    if (!name) return -1;
    for (int o = 0; o < OPT_COUNT; o++)
        if (strcmp(name, kOptions[o].name) == 0) return o;
    return -1;
}
}  // namespace

int option(Option o) {
    init_options();
    return g_options[o].load(std::memory_order_relaxed);
}
int32_t error_flag_ptr(hipStream_t stream, int32_t** out) {
    std::lock_guard<std::mutex> lock(g_mu);
    int32_t*& p = g_error_flags[stream];
    if (!p) {
        DNH_TRY(device_malloc((void**)&p, sizeof(int32_t), "index error word"));
        DNH_HIP(hipMemset(p, 0, sizeof(int32_t)));   // synchronous: done before any kernel that may set it is queued
    }
    *out = p;
    return DNH_OK;
}

int32_t workspace(hipStream_t stream, size_t bytes, void** out, WorkspaceLease& lease) {
    Workspace* w;
    {
        std::lock_guard<std::mutex> lock(g_mu);
        w = &g_ws[stream];   // map nodes do not move
    }
    if (lease.held_ != &w->in_use) {
        lease.release();
        w->in_use.lock();
        lease.held_ = &w->in_use;
    }
    if (w->bytes < bytes) {
        if (w->ptr) {
            // work that still reads the old buffer is ordered before the free by synchronising the stream
            DNH_HIP(hipStreamSynchronize(stream));
            DNH_HIP(hipFree(w->ptr));
            w->ptr = nullptr;
            w->bytes = 0;
        }
        size_t want = bytes < (size_t)(4 << 20) ? (size_t)(4 << 20) : bytes + bytes / 2;
        if (device_malloc(&w->ptr, want, "workspace") != DNH_OK) DNH_TRY(device_malloc(&w->ptr, want = bytes, "workspace"));   // without the head room
        w->bytes = want;
    }
    *out = w->ptr;
    return DNH_OK;
}

__global__ void zero_words_kernel(unsigned long long* p, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0ull;
}

int32_t sync_words(hipStream_t stream, size_t bytes, void** out, uint32_t* epoch, WorkspaceLease& lease) {
    Workspace* w;
    {
        std::lock_guard<std::mutex> lock(g_mu);
        w = &g_ws[stream];
    }
    if (lease.held_ != &w->in_use) {
        lease.release();
        w->in_use.lock();
        lease.held_ = &w->in_use;
    }
    bool clear = false;
    if (w->sync_bytes < bytes) {
        if (w->sync_ptr) {
            DNH_HIP(hipStreamSynchronize(stream));
            DNH_HIP(hipFree(w->sync_ptr));
            w->sync_ptr = nullptr;
            w->sync_bytes = 0;
        }
        const size_t want = (bytes < (size_t)(64 << 10) ? (size_t)(64 << 10) : bytes * 2 + 7) / 8 * 8;
        DNH_TRY(device_malloc(&w->sync_ptr, want, "synchronisation words"));
        w->sync_bytes = want;
        clear = true;
    }
    if (++w->epoch >= (1u << 30)) {
        w->epoch = 1;
        clear = true;
    }
    if (clear) {   // a fill kernel, not a memset node: the call may be under stream capture; ordered before the kernels the caller queues next
        const size_t nwords = w->sync_bytes / 8;
        hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)((nwords + 255) / 256)), dim3(256), 0, stream, (unsigned long long*)w->sync_ptr, nwords);
        DNH_LAUNCH_CHECK();
    }
    *out = w->sync_ptr;
    *epoch = w->epoch;
    return DNH_OK;
}

static void drop_workspace(hipStream_t stream) {
    std::lock_guard<std::mutex> lock(g_mu);
    auto ef = g_error_flags.find(stream);
    if (ef != g_error_flags.end()) {
        if (ef->second) (void)hipFree(ef->second);
        g_error_flags.erase(ef);
    }
    auto it = g_ws.find(stream);
    if (it != g_ws.end()) {
        if (it->second.ptr) (void)hipFree(it->second.ptr);
        if (it->second.sync_ptr) (void)hipFree(it->second.sync_ptr);
        g_ws.erase(it);
    }
}

}  // namespace dnh

using namespace dnh;

extern "C" {

int32_t dnh_init(int32_t device) {
    std::lock_guard<std::mutex> lock(g_mu);
    return init_locked(device);
}

int32_t dnh_device_info(DnhDeviceInfo* info) {
    if (!info) return fail(DNH_ERR_INVALID_ARG, "dnh_device_info: null argument");
    DNH_TRY(ensure_init());
    hipDeviceProp_t prop;
    DNH_HIP(hipGetDeviceProperties(&prop, g_device));
    memset(info, 0, sizeof(*info));
    info->device = g_device;
    info->compute_units = prop.multiProcessorCount;
    info->wavefront_size = prop.warpSize;
    info->max_threads_per_block = prop.maxThreadsPerBlock;
    info->lds_bytes_per_block = (int64_t)prop.sharedMemPerBlock;
    info->total_memory_bytes = (int64_t)prop.totalGlobalMem;
    info->l2_bytes = (int64_t)prop.l2CacheSize;
    info->clock_khz = prop.clockRate;
    info->memory_clock_khz = prop.memoryClockRate;
    strncpy(info->name, prop.name, sizeof(info->name) - 1);
    strncpy(info->arch, prop.gcnArchName, sizeof(info->arch) - 1);
    return DNH_OK;
}

int32_t dnh_set_option(const char* name, int32_t value) {
    const int o = find_option(name);
    if (o < 0) return fail(DNH_ERR_INVALID_ARG, "dnh_set_option: unknown option '%s'", name ? name : "(null)");
    if (value < kOptions[o].lo || value > kOptions[o].hi)
        return fail(DNH_ERR_INVALID_ARG, "dnh_set_option: %s takes %d..%d, not %d", name, kOptions[o].lo, kOptions[o].hi, value);
    init_options();
    g_options[o].store(value, std::memory_order_relaxed);
    return DNH_OK;
}

int32_t dnh_get_option(const char* name, int32_t* value) {
    const int o = find_option(name);
    if (o < 0 || !value) return fail(DNH_ERR_INVALID_ARG, "dnh_get_option: unknown option '%s' or null argument", name ? name : "(null)");
    *value = option((Option)o);
    return DNH_OK;
}

int32_t dnh_last_error(char* buf, size_t n) {
    if (!buf || n == 0) return DNH_ERR_INVALID_ARG;
    const std::string& e = last_error();
    size_t m = e.size() < n - 1 ? e.size() : n - 1;
    memcpy(buf, e.data(), m);
    buf[m] = 0;
    return DNH_OK;
}

int32_t dnh_async_error(void* stream, int32_t* code) {
    if (!code) return fail(DNH_ERR_INVALID_ARG, "dnh_async_error: null argument");
    DNH_TRY(ensure_init());
    int32_t flag = 0;
    DNH_HIP(hipStreamSynchronize((hipStream_t)stream));
    int32_t* dev_flag = nullptr;
    DNH_TRY(error_flag_ptr((hipStream_t)stream, &dev_flag));
    DNH_HIP(hipMemcpy(&flag, dev_flag, sizeof(flag), hipMemcpyDeviceToHost));
    if (flag) DNH_HIP(hipMemset(dev_flag, 0, sizeof(flag)));
    *code = flag ? DNH_ERR_INDEX_OUT_OF_RANGE : DNH_OK;
    if (flag) last_error() = "an index tensor held a position outside the indexed tensor's shape";
    return DNH_OK;
}

int32_t dnh_alloc(size_t bytes, void** out) {
    if (!out) return fail(DNH_ERR_INVALID_ARG, "dnh_alloc: null argument");
    DNH_TRY(ensure_init());
    *out = nullptr;
    return device_malloc(out, bytes ? bytes : 1, "dnh_alloc");
}

int32_t dnh_free(void* ptr) {
    if (!ptr) return DNH_OK;
    DNH_TRY(ensure_init());
    {
        std::lock_guard<std::mutex> lock(g_pool.mu);
        auto it = g_pool.live.find(ptr);
        if (it != g_pool.live.end()) {
            g_pool.live_bytes -= it->second;
            g_pool.live.erase(it);
        }
    }
    DNH_HIP(hipFree(ptr));  // hipFree waits for outstanding work that may still use the buffer
    return DNH_OK;
}

int32_t dnh_alloc_async(size_t bytes, void* stream, void** out) {
    if (!out) return fail(DNH_ERR_INVALID_ARG, "dnh_alloc_async: null argument");
    DNH_TRY(ensure_init());
    *out = nullptr;
    const size_t want = pool_round(bytes);
    std::lock_guard<std::mutex> lock(g_pool.mu);
    auto fs = g_pool.free_blocks.find((hipStream_t)stream);
    if (fs != g_pool.free_blocks.end()) {
        auto it = fs->second.lower_bound(want);
        if (it != fs->second.end() && it->first <= want + want / 4) {  // bounded waste: at most 25 % over the request
            *out = it->second;
            g_pool.live[*out] = it->first;
            g_pool.live_bytes += it->first;
            g_pool.cached_bytes -= it->first;
            fs->second.erase(it);
            g_pool.hits++;
            return DNH_OK;
        }
    }
    g_pool.misses++;
    hipError_t e = hipMalloc(out, want);
    if (e == hipErrorOutOfMemory) {
        // the reference collects garbage and retries (Cuda/CudaUtils.fs:183-194); here the cache is what can be given back
        (void)hipGetLastError();
        DNH_TRY(pool_trim_locked());
        e = hipMalloc(out, want);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        *out = nullptr;
        if (e == hipErrorOutOfMemory)
            return fail(DNH_ERR_OUT_OF_MEMORY, "device memory allocation of %zu MB failed", want >> 20);
        return fail(DNH_ERR_HIP, "hipMalloc(%zu): %s", want, hipGetErrorString(e));
    }
    g_pool.live[*out] = want;
    g_pool.live_bytes += want;
    return DNH_OK;
}

int32_t dnh_free_async(void* ptr, void* stream) {
    if (!ptr) return DNH_OK;
    DNH_TRY(ensure_init());
    size_t bytes = 0;
    {
        std::lock_guard<std::mutex> lock(g_pool.mu);
        auto it = g_pool.live.find(ptr);
        if (it != g_pool.live.end()) {
            bytes = it->second;
            g_pool.live.erase(it);
            g_pool.live_bytes -= bytes;
            if (g_pool.limit_bytes == 0 || g_pool.cached_bytes + bytes <= g_pool.limit_bytes) {
                // a stream that dnh_stream_destroy has already retired (a finalizer running late): everything queued on it has
                // finished, so the block is free for anyone and goes to the default stream's list instead of a dead one
                hipStream_t owner = (hipStream_t)stream;
                {
                    std::lock_guard<std::mutex> dl(g_dead_mu);
                    for (hipStream_t d : g_dead_streams)
                        if (d == owner) owner = nullptr;
                }
                g_pool.free_blocks[owner].emplace(bytes, ptr);
                g_pool.cached_bytes += bytes;
                return DNH_OK;
            }
        }
    }
    DNH_HIP(hipFree(ptr));  // not from the cache, or the cache is full
    return DNH_OK;
}

int32_t dnh_pool_trim(void) {
    DNH_TRY(ensure_init());
    std::lock_guard<std::mutex> lock(g_pool.mu);
    return pool_trim_locked();
}

int32_t dnh_pool_set_limit(size_t bytes) {
    std::lock_guard<std::mutex> lock(g_pool.mu);
    g_pool.limit_bytes = bytes;
    return DNH_OK;
}

int32_t dnh_pool_stats(DnhPoolStats* stats) {
    if (!stats) return fail(DNH_ERR_INVALID_ARG, "dnh_pool_stats: null argument");
    std::lock_guard<std::mutex> lock(g_pool.mu);
    stats->live_bytes = (int64_t)g_pool.live_bytes;
    stats->cached_bytes = (int64_t)g_pool.cached_bytes;
    stats->limit_bytes = (int64_t)g_pool.limit_bytes;
    stats->hits = (int64_t)g_pool.hits;
    stats->misses = (int64_t)g_pool.misses;
    return DNH_OK;
}

int32_t dnh_host_alloc(size_t bytes, void** out) {
    if (!out) return fail(DNH_ERR_INVALID_ARG, "dnh_host_alloc: null argument");
    DNH_TRY(ensure_init());
    *out = nullptr;
    DNH_HIP(hipHostMalloc(out, bytes ? bytes : 1, hipHostMallocDefault));
    {
        std::lock_guard<std::mutex> lock(g_pinned_mu);
        g_pinned[(uintptr_t)*out] = bytes ? bytes : 1;
    }
    return DNH_OK;
}

int32_t dnh_host_free(void* ptr) {
    if (!ptr) return DNH_OK;
    DNH_TRY(ensure_init());
    {
        std::lock_guard<std::mutex> lock(g_pinned_mu);
        g_pinned.erase((uintptr_t)ptr);
    }
    DNH_HIP(hipHostFree(ptr));
    return DNH_OK;
}

int32_t dnh_memset(void* dst, int32_t byte_value, size_t bytes, void* stream) {
    DNH_TRY(ensure_init());
    if (bytes == 0) return DNH_OK;
    DNH_HIP(hipMemsetAsync(dst, byte_value, bytes, (hipStream_t)stream));
    return DNH_OK;
}

// ---- large copies between pageable host memory and the device ------------------------------------------------------------------
// The reference registers host arrays with the driver to copy at the full link rate (Tensor/Tensor/Cuda/CudaRegMem.fs); memory
// that already exists cannot be registered here, and a plain copy from pageable memory runs at a third to a half of the pinned
// rate.  Synchronous copies of 16 MiB and more are therefore staged by the library: a few host threads, each with two pinned
// 4 MiB chunks and a stream of its own, move their share of the chunks (host copy of one chunk while the other is on the link).
namespace {
constexpr size_t kStageChunk = (size_t)4 << 20;
constexpr size_t kStageMin = (size_t)16 << 20;
constexpr int kStageThreads = 6;

struct Stager {
    std::mutex mu;   // one staged copy at a time
    bool ready = false;
    void* pinned[kStageThreads][2] = {};
    hipStream_t stream[kStageThreads] = {};
    hipEvent_t done[kStageThreads][2] = {};
};
Stager g_stager;

bool is_pinned(const void* p, size_t bytes) {
    std::lock_guard<std::mutex> lock(g_pinned_mu);
    auto it = g_pinned.upper_bound((uintptr_t)p);
    if (it == g_pinned.begin()) return false;
    --it;
    return (uintptr_t)p + bytes <= it->first + it->second;
}

int32_t stager_init_locked() {
    if (g_stager.ready) return DNH_OK;
    for (int t = 0; t < kStageThreads; t++) {
        DNH_HIP(hipStreamCreateWithFlags(&g_stager.stream[t], hipStreamNonBlocking));
        for (int k = 0; k < 2; k++) {
            DNH_HIP(hipHostMalloc(&g_stager.pinned[t][k], kStageChunk, hipHostMallocDefault));
            DNH_HIP(hipEventCreateWithFlags(&g_stager.done[t][k], hipEventDisableTiming));
        }
    }
    g_stager.ready = true;
    return DNH_OK;
}

// Worker t moves chunks t, t + kStageThreads, ...; returns the first HIP error it met.
hipError_t stage_worker(int t, bool to_device, char* dev, char* host, size_t bytes) {
    hipError_t e = hipSetDevice(g_device);
    if (e != hipSuccess) return e;
    const size_t chunks = (bytes + kStageChunk - 1) / kStageChunk;
    hipStream_t s = g_stager.stream[t];
    int slot = 0;
    size_t prev_off = 0, prev_len = 0;
    int prev_slot = -1;
    for (size_t i = (size_t)t; i < chunks; i += kStageThreads, slot ^= 1) {
        const size_t off = i * kStageChunk, len = bytes - off < kStageChunk ? bytes - off : kStageChunk;
        void* pin = g_stager.pinned[t][slot];
        if (to_device) {
            if ((e = hipEventSynchronize(g_stager.done[t][slot])) != hipSuccess) return e;   // the chunk's previous transfer has left it
            memcpy(pin, host + off, len);
            if ((e = hipMemcpyAsync(dev + off, pin, len, hipMemcpyHostToDevice, s)) != hipSuccess) return e;
            if ((e = hipEventRecord(g_stager.done[t][slot], s)) != hipSuccess) return e;
        } else {
            if ((e = hipMemcpyAsync(pin, dev + off, len, hipMemcpyDeviceToHost, s)) != hipSuccess) return e;
            if ((e = hipEventRecord(g_stager.done[t][slot], s)) != hipSuccess) return e;
            if (prev_slot >= 0) {
                if ((e = hipEventSynchronize(g_stager.done[t][prev_slot])) != hipSuccess) return e;
                memcpy(host + prev_off, g_stager.pinned[t][prev_slot], prev_len);
            }
            prev_off = off;
            prev_len = len;
            prev_slot = slot;
        }
    }
    if (!to_device && prev_slot >= 0) {
        if ((e = hipEventSynchronize(g_stager.done[t][prev_slot])) != hipSuccess) return e;
        memcpy(host + prev_off, g_stager.pinned[t][prev_slot], prev_len);
    }
    return hipStreamSynchronize(s);
}

int32_t staged_copy(bool to_device, void* dev, void* host, size_t bytes, hipStream_t stream) {
    std::lock_guard<std::mutex> lock(g_stager.mu);
    DNH_TRY(stager_init_locked());
    DNH_HIP(hipStreamSynchronize(stream));   // everything queued before the copy has finished with the device buffer
    hipError_t errs[kStageThreads];
    std::vector<std::thread> workers;
    for (int t = 1; t < kStageThreads; t++)
        workers.emplace_back([&, t] { errs[t] = stage_worker(t, to_device, (char*)dev, (char*)host, bytes); });
    errs[0] = stage_worker(0, to_device, (char*)dev, (char*)host, bytes);
    for (auto& w : workers) w.join();
    for (int t = 0; t < kStageThreads; t++) DNH_HIP(errs[t]);
    return DNH_OK;
}
}  // namespace

static int32_t copy_impl(void* dst, const void* src, size_t bytes, void* stream, int32_t sync, hipMemcpyKind kind) {
    DNH_TRY(ensure_init());
    if (bytes == 0) return DNH_OK;
    if (!dst || !src) return fail(DNH_ERR_INVALID_ARG, "memcpy: null pointer");
    if (sync && bytes >= kStageMin && kind != hipMemcpyDeviceToDevice) {
        const bool to_device = kind == hipMemcpyHostToDevice;
        void* host = to_device ? const_cast<void*>(src) : dst;
        if (!is_pinned(host, bytes)) return staged_copy(to_device, to_device ? dst : const_cast<void*>(src), host, bytes, (hipStream_t)stream);
    }
    DNH_HIP(hipMemcpyAsync(dst, src, bytes, kind, (hipStream_t)stream));
    if (sync) DNH_HIP(hipStreamSynchronize((hipStream_t)stream));
    return DNH_OK;
}

int32_t dnh_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream, int32_t sync) {
    return copy_impl(dst, src, bytes, stream, sync, hipMemcpyHostToDevice);
}
int32_t dnh_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream, int32_t sync) {
    return copy_impl(dst, src, bytes, stream, sync, hipMemcpyDeviceToHost);
}
int32_t dnh_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream, int32_t sync) {
    return copy_impl(dst, src, bytes, stream, sync, hipMemcpyDeviceToDevice);
}

int32_t dnh_stream_create(void** stream) {
    if (!stream) return fail(DNH_ERR_INVALID_ARG, "dnh_stream_create: null argument");
    DNH_TRY(ensure_init());
    hipStream_t s;
    DNH_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    {
        std::lock_guard<std::mutex> dl(g_dead_mu);   // the driver may hand out a retired handle again
        for (size_t i = 0; i < g_dead_streams.size(); i++)
            if (g_dead_streams[i] == s) { g_dead_streams.erase(g_dead_streams.begin() + i); break; }
    }
    *stream = (void*)s;
    return DNH_OK;
}

int32_t dnh_stream_destroy(void* stream) {
    if (!stream) return DNH_OK;
    DNH_TRY(ensure_init());
    DNH_HIP(hipStreamSynchronize((hipStream_t)stream));
    drop_workspace((hipStream_t)stream);
    {
        // everything queued on the stream has finished, so its cached blocks are free for any stream; keep them under
        // the default stream, whose later work is ordered after this point on the host
        std::lock_guard<std::mutex> lock(g_pool.mu);
        auto it = g_pool.free_blocks.find((hipStream_t)stream);
        if (it != g_pool.free_blocks.end()) {
            auto& dflt = g_pool.free_blocks[(hipStream_t) nullptr];
            for (auto& blk : it->second) dflt.emplace(blk.first, blk.second);
            g_pool.free_blocks.erase((hipStream_t)stream);
        }
    }
    DNH_HIP(hipStreamDestroy((hipStream_t)stream));
    {
        std::lock_guard<std::mutex> dl(g_dead_mu);
        g_dead_streams.push_back((hipStream_t)stream);
    }
    return DNH_OK;
}

int32_t dnh_stream_sync(void* stream) {
    DNH_TRY(ensure_init());
    DNH_HIP(hipStreamSynchronize((hipStream_t)stream));
    return DNH_OK;
}

int32_t dnh_device_sync(void) {
    DNH_TRY(ensure_init());
    DNH_HIP(hipDeviceSynchronize());
    return DNH_OK;
}

int32_t dnh_event_create(void** event) {
    if (!event) return fail(DNH_ERR_INVALID_ARG, "dnh_event_create: null argument");
    DNH_TRY(ensure_init());
    hipEvent_t e;
    DNH_HIP(hipEventCreate(&e));
    *event = (void*)e;
    return DNH_OK;
}
int32_t dnh_event_destroy(void* event) {
    if (!event) return DNH_OK;
    DNH_TRY(ensure_init());
    DNH_HIP(hipEventDestroy((hipEvent_t)event));
    return DNH_OK;
}
int32_t dnh_event_record(void* event, void* stream) {
    DNH_TRY(ensure_init());
    DNH_HIP(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
    return DNH_OK;
}
int32_t dnh_event_sync(void* event) {
    DNH_TRY(ensure_init());
    DNH_HIP(hipEventSynchronize((hipEvent_t)event));
    return DNH_OK;
}
int32_t dnh_event_elapsed_ms(void* start, void* stop, float* ms) {
    if (!ms) return fail(DNH_ERR_INVALID_ARG, "dnh_event_elapsed_ms: null argument");
    DNH_TRY(ensure_init());
    DNH_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return DNH_OK;
}

}  // extern "C"
