// Device runtime shim of the C ABI: device selection, a caching allocator,
// copies, streams, events and the error text.
#include "rp_common.h"

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

namespace rp {

static thread_local char g_error[512] = "";
static thread_local hipStream_t g_stream = nullptr;

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    if (getenv("RP_HIP_VERBOSE")) fprintf(stderr, "rp_hip: %s\n", g_error);
}

hipStream_t current_stream() { flush_deferred(); return g_stream; }

bool check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return true;
    set_error("%s: %s", what, hipGetErrorString(e));
    return false;
}

bool check_launch(const char* what) { return check_hip(hipGetLastError(), what); }

int device_cu_count() {
    constexpr int MAX_DEVICES = 64;
    static std::atomic<int> cached[MAX_DEVICES] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) { (void)hipGetLastError(); return 0; }
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) { (void)hipGetLastError(); n = 0; }
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

bool path_disabled(const char* name) {
    static const std::string list = [] { const char* e = getenv("RP_HIP_DISABLE"); return std::string(",") + (e ? e : "") + ","; }();
    return list.find(std::string(",") + name + ",") != std::string::npos;
}

// ---- workgroup placement -----------------------------------------------------
// The dispatcher deals the workgroups of a grid to the XCDs round robin, so workgroups b and b + 8 share an L2.
// Kernels that exchange data between workgroups through that L2 rely on it, so it is observed rather than assumed:
// every workgroup of a 1 024-block grid records the XCC it runs on, three launches in a row, and the rule must
// hold for all of them.  (A device with a single XCD passes trivially.)  The record lives in a device array of the
// library, so the check allocates nothing.
constexpr int PLACEMENT_BLOCKS = 1024;
static __device__ int g_xcc_of_block[PLACEMENT_BLOCKS];

__global__ void __launch_bounds__(256) record_xcc_kernel() {
    if (threadIdx.x == 0) {
        unsigned xcc;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
        g_xcc_of_block[blockIdx.x] = (int)(xcc & 15u);
    }
}

bool workgroups_share_xcd_by_residue() {
    constexpr int MAX_DEVICES = 64;
    static std::atomic<int> state[MAX_DEVICES] = {};          // 0 unknown, 1 holds, 2 does not
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) { (void)hipGetLastError(); return false; }
    int st = state[dev].load(std::memory_order_acquire);
    if (st != 0) return st == 1;
    if (stream_is_capturing()) return false;
    static std::mutex mu;
    std::lock_guard<std::mutex> lock(mu);
    st = state[dev].load(std::memory_order_acquire);
    if (st != 0) return st == 1;
    bool holds = !path_disabled("l2_exchange");
    static int seen[PLACEMENT_BLOCKS];
    for (int rep = 0; rep < 3 && holds; rep++) {
        hipLaunchKernelGGL(record_xcc_kernel, dim3(PLACEMENT_BLOCKS), dim3(256), 0, current_stream());
        if (hipGetLastError() != hipSuccess || hipStreamSynchronize(current_stream()) != hipSuccess ||
            hipMemcpyFromSymbol(seen, HIP_SYMBOL(g_xcc_of_block), sizeof(seen)) != hipSuccess) { (void)hipGetLastError(); return false; }   // not decided: ask again later
        for (int b = 8; b < PLACEMENT_BLOCKS; b++) holds = holds && seen[b] == seen[b % 8];
    }
    state[dev].store(holds ? 1 : 2, std::memory_order_release);
    return holds;
}

// ---- caching allocator ------------------------------------------------------
// The reference allocates and zero-fills device memory for every op output
// (core/tensor_device.cu:44-46) and frees it when the tensor dies; hipMalloc /
// hipFree cost tens of microseconds and hipFree synchronises the device, which
// would dominate the small-GEMM configs.  Freed blocks are therefore kept per
// device in size-keyed lists and reused.  The lists are shared by every thread
// and stream of the process: a block freed while kernels that use it are still
// queued may be handed to the very next rp_hip_malloc of its size, which is safe
// for work issued afterwards on the same stream only.  Callers that run several
// streams at once wait for a block's last user before freeing it.
struct Pool {
    std::mutex mu;
    std::unordered_map<void*, std::pair<int, size_t>> live;       // ptr -> (device, rounded size)
    std::map<std::pair<int, size_t>, std::vector<void*>> free_lists;
    bool enabled = true;
    Pool() { const char* e = getenv("RP_HIP_NO_CACHE"); enabled = !(e && e[0] == '1'); }
};

static Pool& pool() { static Pool* p = new Pool(); return *p; }   // leaked on purpose: outlives HIP teardown

// what rp_hip_memory_stats reports: requests to rp_hip_malloc, and how many of them reached hipMalloc
static std::atomic<long long> g_malloc_requests{0}, g_device_mallocs{0};

// Blocks and graph capture.  A kernel recorded into a graph keeps the addresses it was recorded with, so a block
// that is freed while the calling thread records (a split-k workspace, an intermediate tensor) must not be handed
// to anyone else for as long as the graph can be replayed: every replay writes there.  While a capture that this
// library began is active, freed blocks therefore go to a list of the capture (later allocations of the same
// capture may take them again, which is the stream-ordered reuse the recording itself has); at the capture's end
// the list is tied to the executable graph, and rp_hip_graph_destroy gives the blocks back to the pool.
// rp_hip_empty_cache only sees the pool's own lists, so it never releases such a block.
struct HeldBlock { void* ptr; int dev; size_t size; };
struct CaptureState { bool active = false; std::vector<HeldBlock> freed; };
static thread_local CaptureState g_capture;
static std::mutex g_graph_mu;
static std::unordered_map<void*, std::vector<HeldBlock>>& graph_blocks() { static auto* m = new std::unordered_map<void*, std::vector<HeldBlock>>(); return *m; }

static void release_to_pool(const std::vector<HeldBlock>& blocks) {
    Pool& p = pool();
    for (const HeldBlock& b : blocks) {
        if (p.enabled) { std::lock_guard<std::mutex> lk(p.mu); p.free_lists[{b.dev, b.size}].push_back(b.ptr); }
        else (void)hipFree(b.ptr);
    }
}

// true when the calling thread's stream is recording a graph that was not begun through this library
static bool foreign_capture() {
    if (!g_stream || g_capture.active) return false;
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(g_stream, &st) != hipSuccess) { (void)hipGetLastError(); return false; }
    return st != hipStreamCaptureStatusNone;
}

bool stream_is_capturing() { return g_capture.active || foreign_capture(); }

static size_t round_size(size_t bytes) {
    if (bytes == 0) bytes = 1;
    if (bytes <= (1u << 20)) return (bytes + 511) & ~(size_t)511;          // 512 B steps up to 1 MiB
    return (bytes + ((1u << 21) - 1)) & ~(size_t)((1u << 21) - 1);         // 2 MiB steps above
}

struct SmallPayload { uint32_t w[512]; };            // 2 KiB, passed by value in the kernel arguments
__global__ void upload_small_kernel(uint32_t* dst, SmallPayload payload, int nwords) {
    int i = blockIdx.x * 256 + threadIdx.x;
    if (i < nwords) dst[i] = payload.w[i];
}

// Byte fill: a 16-byte aligned body written as uint4 plus scalar head and tail.
__global__ void fill_bytes_kernel(unsigned char* p, unsigned char v, size_t bytes) {
    size_t head = (16 - ((uintptr_t)p & 15)) & 15;
    if (head > bytes) head = bytes;
    size_t body = (bytes - head) / 16;
    size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t nth = (size_t)gridDim.x * blockDim.x;
    uint32_t w = 0x01010101u * v;
    uint4 w4 = make_uint4(w, w, w, w);
    uint4* q = (uint4*)(p + head);
    for (size_t i = tid; i < body; i += nth) q[i] = w4;
    size_t tail0 = head + body * 16;
    for (size_t i = tid; i < head; i += nth) p[i] = v;
    for (size_t i = tail0 + tid; i < bytes; i += nth) p[i] = v;
}

}  // namespace rp

using namespace rp;

extern "C" {

int rp_hip_device_count(int* count) {
    if (!count) { set_error("rp_hip_device_count: null argument"); return -1; }
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) { (void)hipGetLastError(); n = 0; }       // no device is an answer, not a failure
    *count = n;
    return 0;
}

int rp_hip_set_device(int device_id) {
    int cur = -1;
    if (hipGetDevice(&cur) != hipSuccess) { (void)hipGetLastError(); cur = -1; }
    if (cur != device_id) flush_deferred();             // a postponed multiply belongs to the device it was recorded on
    return check_hip(hipSetDevice(device_id), "hipSetDevice") ? 0 : -1;
}

int rp_hip_get_device(int* device_id) {
    if (!device_id) { set_error("rp_hip_get_device: null argument"); return -1; }
    return check_hip(hipGetDevice(device_id), "hipGetDevice") ? 0 : -1;
}

int rp_hip_malloc(void** ptr, size_t bytes) {
    if (!ptr) { set_error("rp_hip_malloc: null argument"); return -1; }
    *ptr = nullptr;
    g_malloc_requests.fetch_add(1, std::memory_order_relaxed);
    int dev = 0;
    if (!check_hip(hipGetDevice(&dev), "hipGetDevice")) return -1;
    Pool& p = pool();
    size_t sz = round_size(bytes);
    if (g_capture.active) {                          // a block this recording has already let go of
        for (size_t i = g_capture.freed.size(); i-- > 0;) {
            const HeldBlock b = g_capture.freed[i];
            if (b.dev != dev || b.size != sz) continue;
            g_capture.freed.erase(g_capture.freed.begin() + (long)i);
            std::lock_guard<std::mutex> lk(p.mu);
            p.live[b.ptr] = {dev, sz};
            *ptr = b.ptr;
            return 0;
        }
    }
    if (p.enabled) {
        std::lock_guard<std::mutex> lk(p.mu);
        auto it = p.free_lists.find({dev, sz});
        if (it != p.free_lists.end() && !it->second.empty()) {
            *ptr = it->second.back();
            it->second.pop_back();
            p.live[*ptr] = {dev, sz};
            return 0;
        }
    }
    void* d = nullptr;
    g_device_mallocs.fetch_add(1, std::memory_order_relaxed);
    hipError_t e = hipMalloc(&d, sz);
    if (e != hipSuccess && p.enabled) {            // out of memory: give cached blocks back and retry once
        (void)hipGetLastError();
        rp_hip_empty_cache();
        e = hipMalloc(&d, sz);
    }
    if (!check_hip(e, "hipMalloc")) return -1;
    {
        std::lock_guard<std::mutex> lk(p.mu);
        p.live[d] = {dev, sz};
    }
    *ptr = d;
    return 0;
}

int rp_hip_free(void* ptr) {
    if (!ptr) return 0;
    if (deferred_touches(ptr)) flush_deferred();        // a postponed multiply still uses the block: it runs first, in stream order before any reuse
    Pool& p = pool();
    {
        std::lock_guard<std::mutex> lk(p.mu);
        auto it = p.live.find(ptr);
        if (it == p.live.end()) { set_error("rp_hip_free: pointer %p was not allocated by rp_hip_malloc", ptr); return -1; }
        auto key = it->second;
        p.live.erase(it);
        if (g_capture.active) { g_capture.freed.push_back({ptr, key.first, key.second}); return 0; }    // stays with the graph being recorded
        if (foreign_capture()) {
            // recorded by a graph this library knows nothing about: the block is never handed out again
            std::lock_guard<std::mutex> gl(g_graph_mu);
            graph_blocks()[nullptr].push_back({ptr, key.first, key.second});
            return 0;
        }
        if (p.enabled) { p.free_lists[key].push_back(ptr); return 0; }
    }
    return check_hip(hipFree(ptr), "hipFree") ? 0 : -1;
}

int rp_hip_memory_stats(long long* malloc_requests, long long* device_mallocs, long long* live_blocks, long long* cached_blocks) {
    Pool& p = pool();
    if (malloc_requests) *malloc_requests = g_malloc_requests.load(std::memory_order_relaxed);
    if (device_mallocs) *device_mallocs = g_device_mallocs.load(std::memory_order_relaxed);
    std::lock_guard<std::mutex> lk(p.mu);
    if (live_blocks) *live_blocks = (long long)p.live.size();
    if (cached_blocks) { long long n = 0; for (auto& kv : p.free_lists) n += (long long)kv.second.size(); *cached_blocks = n; }
    return 0;
}

int rp_hip_empty_cache(void) {
    Pool& p = pool();
    std::vector<void*> blocks;
    {
        std::lock_guard<std::mutex> lk(p.mu);
        for (auto& kv : p.free_lists) for (void* b : kv.second) blocks.push_back(b);
        p.free_lists.clear();
    }
    bool ok = true;
    for (void* b : blocks) ok = check_hip(hipFree(b), "hipFree") && ok;
    return ok ? 0 : -1;
}

// A fill kernel rather than hipMemsetAsync, so the call can be captured into a
// HIP graph by callers that record their step.
int rp_hip_memset(void* ptr, int value, size_t bytes) {
    if (!ptr && bytes) { set_error("rp_hip_memset: null pointer"); return -1; }
    if (!bytes) return 0;
    size_t per_block = (size_t)256 * 16;
    size_t blocks = (bytes + per_block - 1) / per_block;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(rp::fill_bytes_kernel, dim3((unsigned)blocks), dim3(256), 0, current_stream(),
                       (unsigned char*)ptr, (unsigned char)value, bytes);
    return check_launch("fill_bytes_kernel") ? 0 : -1;
}

// Host copies block until the data has landed, like the reference's cudaMemcpy
// calls (core/tensor_device.cu:295-531); device-to-device copies are stream-ordered.
// Exception: a host-to-device copy of at most 2 KiB of whole words travels inside a
// kernel's arguments.  The source is read before the call returns and the data is
// in place for everything that follows on the stream, which is all a caller of
// cudaMemcpy can observe, but the host does not wait for the stream to drain (class
// targets uploaded between a forward and a backward pass would otherwise stall both).
int rp_hip_memcpy_h2d(void* dst, const void* src, size_t bytes) {
    if (!bytes) return 0;
    if (!dst || !src) { set_error("rp_hip_memcpy_h2d: null pointer"); return -1; }
    if (bytes <= sizeof(rp::SmallPayload) && bytes % 4 == 0 && ((uintptr_t)dst & 3) == 0) {
        rp::SmallPayload payload;
        memcpy(payload.w, src, bytes);
        const int nwords = (int)(bytes / 4);
        hipLaunchKernelGGL(rp::upload_small_kernel, dim3((nwords + 255) / 256), dim3(256), 0, current_stream(), (uint32_t*)dst, payload, nwords);
        return check_launch("upload_small_kernel") ? 0 : -1;
    }
    if (!check_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, current_stream()), "hipMemcpy H2D")) return -1;
    return check_hip(hipStreamSynchronize(current_stream()), "hipStreamSynchronize") ? 0 : -1;
}

int rp_hip_memcpy_d2h(void* dst, const void* src, size_t bytes) {
    if (!bytes) return 0;
    if (!dst || !src) { set_error("rp_hip_memcpy_d2h: null pointer"); return -1; }
    if (!check_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, current_stream()), "hipMemcpy D2H")) return -1;
    return check_hip(hipStreamSynchronize(current_stream()), "hipStreamSynchronize") ? 0 : -1;
}

int rp_hip_memcpy_d2d(void* dst, const void* src, size_t bytes) {
    if (!bytes) return 0;
    if (!dst || !src) { set_error("rp_hip_memcpy_d2d: null pointer"); return -1; }
    return check_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, current_stream()), "hipMemcpy D2D") ? 0 : -1;
}

int rp_hip_synchronize(void) {
    flush_deferred();
    return check_hip(hipDeviceSynchronize(), "hipDeviceSynchronize") ? 0 : -1;
}

const char* rp_hip_last_error(void) { return g_error; }

int rp_hip_set_stream(void* stream) { flush_deferred(); g_stream = (hipStream_t)stream; return 0; }      // (a postponed multiply belongs to the stream it was recorded on)
void* rp_hip_get_stream(void) { flush_deferred(); return (void*)g_stream; }                               // (the caller may launch work of its own on it)

int rp_hip_stream_create(void** stream) {
    if (!stream) { set_error("rp_hip_stream_create: null argument"); return -1; }
    hipStream_t st;
    if (!check_hip(hipStreamCreateWithFlags(&st, hipStreamNonBlocking), "hipStreamCreate")) return -1;   // default priority
    *stream = (void*)st;
    return 0;
}

int rp_hip_stream_destroy(void* stream) {
    if (g_stream == (hipStream_t)stream) g_stream = nullptr;
    return check_hip(hipStreamDestroy((hipStream_t)stream), "hipStreamDestroy") ? 0 : -1;
}

int rp_hip_stream_synchronize(void) {
    return check_hip(hipStreamSynchronize(current_stream()), "hipStreamSynchronize") ? 0 : -1;
}

// Record everything the calling thread enqueues on its current stream (which must be a created stream, not
// the null stream) into a graph.  Entry points of this library launch kernels only (clears are fill kernels,
// not memset nodes), so a recorded sequence replays exactly; host-blocking copies must stay outside.
int rp_hip_graph_capture_begin(void) {
    if (!g_stream) { set_error("rp_hip_graph_capture_begin: set a created stream first (the null stream cannot be captured)"); return -1; }
    if (g_capture.active) { set_error("rp_hip_graph_capture_begin: this thread is already recording"); return -1; }
    flush_deferred();                                   // work asked for before the recording stays outside it
    if (!check_hip(hipStreamBeginCapture(g_stream, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture")) return -1;
    g_capture.active = true;
    g_capture.freed.clear();
    return 0;
}

int rp_hip_graph_capture_end(void** graph_exec) {
    if (!graph_exec) { set_error("rp_hip_graph_capture_end: null argument"); return -1; }
    hipGraph_t graph = nullptr;
    flush_deferred();                                   // and work asked for inside it is part of it
    std::vector<HeldBlock> held;
    held.swap(g_capture.freed);
    g_capture.active = false;
    if (!check_hip(hipStreamEndCapture(g_stream, &graph), "hipStreamEndCapture")) { release_to_pool(held); return -1; }
    hipGraphExec_t exec = nullptr;
    bool ok = check_hip(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0), "hipGraphInstantiate");
    (void)hipGraphDestroy(graph);
    if (!ok) { release_to_pool(held); return -1; }       // nothing can replay the recording
    if (!held.empty()) { std::lock_guard<std::mutex> gl(g_graph_mu); graph_blocks()[(void*)exec] = std::move(held); }
    *graph_exec = (void*)exec;
    return 0;
}

int rp_hip_graph_launch(void* graph_exec) {
    return check_hip(hipGraphLaunch((hipGraphExec_t)graph_exec, current_stream()), "hipGraphLaunch") ? 0 : -1;
}

int rp_hip_graph_destroy(void* graph_exec) {
    if (!graph_exec) return 0;
    const bool ok = check_hip(hipGraphExecDestroy((hipGraphExec_t)graph_exec), "hipGraphExecDestroy");
    std::vector<HeldBlock> held;
    {
        std::lock_guard<std::mutex> gl(g_graph_mu);
        auto it = graph_blocks().find(graph_exec);
        if (it != graph_blocks().end()) { held = std::move(it->second); graph_blocks().erase(it); }
    }
    release_to_pool(held);          // the caller has waited for the last replay, as before any free
    return ok ? 0 : -1;
}

int rp_hip_event_create(void** event) {
    if (!event) { set_error("rp_hip_event_create: null argument"); return -1; }
    hipEvent_t ev;
    if (!check_hip(hipEventCreate(&ev), "hipEventCreate")) return -1;
    *event = (void*)ev;
    return 0;
}

int rp_hip_event_record(void* event) {
    return check_hip(hipEventRecord((hipEvent_t)event, current_stream()), "hipEventRecord") ? 0 : -1;
}

int rp_hip_event_synchronize(void* event) {
    return check_hip(hipEventSynchronize((hipEvent_t)event), "hipEventSynchronize") ? 0 : -1;
}

int rp_hip_event_elapsed_ms(float* ms, void* start, void* stop) {
    if (!ms) { set_error("rp_hip_event_elapsed_ms: null argument"); return -1; }
    return check_hip(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop), "hipEventElapsedTime") ? 0 : -1;
}

int rp_hip_event_destroy(void* event) {
    return check_hip(hipEventDestroy((hipEvent_t)event), "hipEventDestroy") ? 0 : -1;
}

}  // extern "C"
