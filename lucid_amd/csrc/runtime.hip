// Runtime entry points of the C ABI: device selection, storage, transfers,
// events, the op registry and synthetic-data fills.
#include <cstring>
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "common.hpp"

namespace lq {

std::string& last_error() {
    thread_local std::string msg;
    return msg;
}

int fail(int status, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    last_error() = buf;
    return status;
}

int hip_fail(hipError_t e, const char* what) {
    int status = LQ_ERR_INTERNAL;
    if (e == hipErrorOutOfMemory) status = LQ_ERR_OOM;
    if (e == hipErrorNoDevice || e == hipErrorInvalidDevice) status = LQ_ERR_GPU_NOT_AVAILABLE;
    return fail(status, "%s: %s", what, hipGetErrorString(e));
}

namespace {
constexpr int kMaxDevices = 16;

// One lock for the runtime's host-side state: the per-stream scratch buffers, the
// caching pool and the graph tables (a scratch request asks whether graphs are
// alive, and destroying a graph releases retired scratch, so separate locks
// would have to nest both ways).
std::recursive_mutex g_rt_mutex;

// ---- per-(device, stream) scratch
// Reduction partials, the im2col fallback's matrix and the split-K slabs live in
// buffers owned by the library.  They are keyed by the stream the call runs on,
// so calls on different streams never share one (calls that overlap on ONE
// stream's buffer are ordered by that stream).  A buffer only ever grows.  The
// block it outgrows is not freed on the spot: a captured graph may have its
// address baked into kernel nodes, and freeing needs a device-wide
// synchronisation that is illegal while a stream is capturing.  Outgrown blocks
// are retired and released at the next moment when no graph exists and nothing
// is being captured.
struct StreamBuf {
    void* ptr = nullptr;
    size_t size = 0;
};
struct BufKey {
    int dev;
    hipStream_t stream;
    int kind;
    bool operator<(const BufKey& o) const {
        if (dev != o.dev) return dev < o.dev;
        if (stream != o.stream) return stream < o.stream;
        return kind < o.kind;
    }
};
std::map<BufKey, StreamBuf> g_bufs;
std::vector<void*> g_retired;

// ---- graphs (tables; the entry points are further down)
struct GraphRec {
    hipGraph_t graph = nullptr;      // the captured template, kept until the exec is destroyed
    hipGraphExec_t exec = nullptr;   // null while capturing or after a failed end
    std::vector<std::pair<int, void*>> blocks;  // (device, block) allocated during capture
    bool capturing = false;          // between a successful begin and its end / destroy
};
std::unordered_map<int, GraphRec> g_graphs;
int g_captures_in_progress = 0;  // records with `capturing` set; changed only together with that flag
int g_next_graph_id = 1;
thread_local int t_capturing_graph = 0;  // id of the graph this thread is capturing, 0 = none

// caller holds g_rt_mutex
bool graphs_quiescent() { return g_graphs.empty() && g_captures_in_progress == 0; }

// caller holds g_rt_mutex.  Frees retired scratch when nothing can still refer to it.
void drain_retired() {
    if (g_retired.empty() || !graphs_quiescent()) return;
    if (hipDeviceSynchronize() != hipSuccess) return;  // keep them; try again later
    for (void* p : g_retired) (void)hipFree(p);
    g_retired.clear();
}
}  // namespace

int stream_buffer(int kind, size_t nbytes, size_t min_bytes, hipStream_t stream, void** ptr, bool* fresh) {
    int dev = 0;
    LQ_HIP(hipGetDevice(&dev));
    LQ_REQUIRE(dev >= 0 && dev < kMaxDevices, LQ_ERR_DEVICE, "device index %d out of range", dev);
    std::lock_guard<std::recursive_mutex> lock(g_rt_mutex);
    StreamBuf& b = g_bufs[BufKey{dev, stream, kind}];
    if (fresh) *fresh = false;
    if (b.size < nbytes || b.ptr == nullptr) {
        const size_t want = nbytes < min_bytes ? min_bytes : nbytes;
        void* p = nullptr;
        LQ_HIP(hipMalloc(&p, want));  // legal during a relaxed capture; no synchronisation here
        if (b.ptr) g_retired.push_back(b.ptr);
        b.ptr = p;
        b.size = want;
        if (fresh) *fresh = true;
        drain_retired();
    }
    *ptr = b.ptr;
    return LQ_OK;
}

int workspace(size_t nbytes, hipStream_t stream, void** ptr) {
    return stream_buffer(0, nbytes, size_t(4) << 20, stream, ptr, nullptr);
}

}  // namespace lq

using namespace lq;

extern "C" {

int lq_version(void) { return LQ_VERSION; }

const char* lq_last_error(void) { return last_error().c_str(); }

int lq_device_count(int* count) {
    LQ_REQUIRE(count, LQ_ERR_VALUE, "count is NULL");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        *count = 0;
        return hip_fail(e, "hipGetDeviceCount");
    }
    *count = n;
    return LQ_OK;
}

int lq_init(int device) {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0)
        return fail(LQ_ERR_GPU_NOT_AVAILABLE, "no HIP device is visible (%s)",
                    e == hipSuccess ? "count = 0" : hipGetErrorString(e));
    LQ_REQUIRE(device >= 0 && device < n, LQ_ERR_DEVICE, "device %d out of range [0,%d)", device, n);
    LQ_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    LQ_HIP(hipGetDeviceProperties(&prop, device));
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(LQ_ERR_GPU_NOT_AVAILABLE, "device %d is %s; this library is built for gfx950 only",
                    device, prop.gcnArchName);
    void* ws = nullptr;
    int rc = workspace(size_t(4) << 20, nullptr, &ws);
    if (rc) return rc;
    return minmax_noalloc_init();  // resolves the static scratch of lq_minmax_noalloc on this device
}

int lq_device_name(char* buf, size_t buflen) {
    LQ_REQUIRE(buf && buflen > 0, LQ_ERR_VALUE, "buf is NULL");
    int dev = 0;
    LQ_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    LQ_HIP(hipGetDeviceProperties(&prop, dev));
    snprintf(buf, buflen, "%s (%s, %d CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
    return LQ_OK;
}

// ------------------------------------------------------------------ caching allocator
// hipMalloc / hipFree cost tens of microseconds and synchronise; a quantized
// model allocates one output per layer.  Freed blocks are therefore kept in
// per-device free lists keyed by their (rounded) size and handed out again.
// Blocks are recycled in submission order, which is safe for work issued on
// one stream; a caller that frees memory still in use on ANOTHER stream must
// synchronise first (as with any pooled allocator).
// While a thread captures a graph (lq_graph_begin .. lq_graph_end) every block
// it allocates is pinned to that graph: replays write into it, so it cannot be
// handed to anyone else before the graph is destroyed.  lq_free on a pinned
// block only records that its owner is done with it; lq_graph_destroy releases
// the blocks so marked and unpins the others, whose owners release them later.
namespace {
struct Pin {
    int graph;
    bool owner_freed;
};
struct Pool {
    std::multimap<size_t, void*> free_blocks;           // size -> block
    std::unordered_map<void*, size_t> live;              // block -> size
    std::unordered_map<void*, Pin> pinned;               // block -> graph that replays into it
    size_t bytes_reserved = 0, bytes_in_use = 0;
};
Pool g_pool[kMaxDevices];

size_t round_size(size_t n) {
    if (n < 512) return 512;
    if (n < (size_t(1) << 20)) return (n + 511) / 512 * 512;
    return (n + (size_t(2) << 20) - 1) / (size_t(2) << 20) * (size_t(2) << 20);  // 2 MiB granules
}
}  // namespace

extern "C" int lq_alloc(void** ptr, size_t nbytes) {
    LQ_REQUIRE(ptr, LQ_ERR_VALUE, "ptr is NULL");
    *ptr = nullptr;
    int dev = 0;
    LQ_HIP(hipGetDevice(&dev));
    LQ_REQUIRE(dev >= 0 && dev < kMaxDevices, LQ_ERR_DEVICE, "device index %d out of range", dev);
    const size_t size = round_size(nbytes);
    std::lock_guard<std::recursive_mutex> lock(g_rt_mutex);
    Pool& pool = g_pool[dev];
    void* p = nullptr;
    auto it = pool.free_blocks.lower_bound(size);
    // reuse a cached block unless it would waste more than half of itself
    if (it != pool.free_blocks.end() && it->first <= size * 2) {
        p = it->second;
        pool.live[p] = it->first;
        pool.bytes_in_use += it->first;
        pool.free_blocks.erase(it);
    } else {
        hipError_t e = hipMalloc(&p, size);
        if (e == hipErrorOutOfMemory) {
            // give cached blocks back to the driver and try once more
            for (auto& kv : pool.free_blocks) (void)hipFree(kv.second);
            for (auto& kv : pool.free_blocks) pool.bytes_reserved -= kv.first;
            pool.free_blocks.clear();
            (void)hipGetLastError();
            e = hipMalloc(&p, size);
        }
        if (e != hipSuccess) return hip_fail(e, "hipMalloc");
        pool.live[p] = size;
        pool.bytes_reserved += size;
        pool.bytes_in_use += size;
    }
    if (t_capturing_graph) {
        pool.pinned[p] = Pin{t_capturing_graph, false};
        g_graphs[t_capturing_graph].blocks.push_back({dev, p});
    }
    *ptr = p;
    return LQ_OK;
}

namespace {
// caller holds g_rt_mutex
void release_block(Pool& pool, void* p) {
    auto it = pool.live.find(p);
    if (it == pool.live.end()) return;
    pool.bytes_in_use -= it->second;
    pool.free_blocks.insert({it->second, p});
    pool.live.erase(it);
}

// caller holds g_rt_mutex.  The graph no longer replays into its blocks: those whose
// owner has already freed them go back to the pool, the others are merely unpinned.
void unpin_graph_blocks(GraphRec& rec) {
    for (auto& db : rec.blocks) {
        Pool& pool = g_pool[db.first];
        auto it = pool.pinned.find(db.second);
        if (it == pool.pinned.end()) continue;
        const bool freed = it->second.owner_freed;
        pool.pinned.erase(it);
        if (freed) release_block(pool, db.second);
    }
    rec.blocks.clear();
}
}  // namespace

extern "C" int lq_free(void* ptr) {
    if (!ptr) return LQ_OK;
    std::lock_guard<std::recursive_mutex> lock(g_rt_mutex);
    for (int dev = 0; dev < kMaxDevices; ++dev) {
        Pool& pool = g_pool[dev];
        if (!pool.live.count(ptr)) continue;
        auto pin = pool.pinned.find(ptr);
        if (pin != pool.pinned.end()) {
            pin->second.owner_freed = true;  // released when its graph is destroyed
            return LQ_OK;
        }
        release_block(pool, ptr);
        return LQ_OK;
    }
    return fail(LQ_ERR_VALUE, "lq_free: pointer %p was not allocated by lq_alloc", ptr);
}

extern "C" int lq_empty_cache(void) {
    LQ_HIP(hipDeviceSynchronize());
    std::lock_guard<std::recursive_mutex> lock(g_rt_mutex);
    int dev = 0;
    LQ_HIP(hipGetDevice(&dev));
    Pool& pool = g_pool[dev];
    for (auto& kv : pool.free_blocks) {
        LQ_HIP(hipFree(kv.second));
        pool.bytes_reserved -= kv.first;
    }
    pool.free_blocks.clear();
    drain_retired();
    return LQ_OK;
}

extern "C" int lq_device_memory_info(size_t* free_bytes, size_t* total_bytes) {
    LQ_REQUIRE(free_bytes && total_bytes, LQ_ERR_VALUE, "device_memory_info: NULL pointer");
    LQ_HIP(hipMemGetInfo(free_bytes, total_bytes));
    return LQ_OK;
}

extern "C" int lq_memory_stats(size_t* bytes_in_use, size_t* bytes_reserved) {
    int dev = 0;
    LQ_HIP(hipGetDevice(&dev));
    std::lock_guard<std::recursive_mutex> lock(g_rt_mutex);
    if (bytes_in_use) *bytes_in_use = g_pool[dev].bytes_in_use;
    if (bytes_reserved) *bytes_reserved = g_pool[dev].bytes_reserved;
    return LQ_OK;
}

// ------------------------------------------------------------------ graphs
// Capture state is per thread (the thread that begins a capture is the one that
// launches into it), so allocations made meanwhile by other threads are not
// pinned to the graph.
extern "C" int lq_graph_begin(lq_stream stream, int* graph_id) {
    LQ_REQUIRE(stream, LQ_ERR_VALUE, "graph capture needs a created stream, not the default stream");
    LQ_REQUIRE(graph_id, LQ_ERR_VALUE, "graph_id is NULL");
    LQ_REQUIRE(t_capturing_graph == 0, LQ_ERR_VALUE, "this thread is already capturing a graph");
    int id = 0;
    {
        std::lock_guard<std::recursive_mutex> lock(g_rt_mutex);
        id = g_next_graph_id++;
        g_graphs[id].capturing = true;
        ++g_captures_in_progress;
    }
    hipError_t e = hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeRelaxed);
    if (e != hipSuccess) {
        std::lock_guard<std::recursive_mutex> lock(g_rt_mutex);
        g_graphs.erase(id);
        --g_captures_in_progress;
        return hip_fail(e, "hipStreamBeginCapture");
    }
    t_capturing_graph = id;
    *graph_id = id;
    return LQ_OK;
}

// On failure the graph id stays known (with no executable) until lq_graph_destroy,
// but the blocks allocated during the capture are unpinned at once.
extern "C" int lq_graph_end(lq_stream stream, int graph_id) {
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(as_stream(stream), &graph);
    if (t_capturing_graph == graph_id) t_capturing_graph = 0;
    hipGraphExec_t exec = nullptr;
    hipError_t e2 = hipSuccess;
    if (e == hipSuccess) e2 = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    std::lock_guard<std::recursive_mutex> lock(g_rt_mutex);
    auto it = g_graphs.find(graph_id);
    // only this record's own capture ends here: a stray or repeated call for another id must not
    // make a capture that is still running look finished
    if (it != g_graphs.end() && it->second.capturing) {
        it->second.capturing = false;
        --g_captures_in_progress;
    }
    if (e != hipSuccess || e2 != hipSuccess || it == g_graphs.end()) {
        if (graph) (void)hipGraphDestroy(graph);
        if (exec) (void)hipGraphExecDestroy(exec);
        if (it != g_graphs.end()) unpin_graph_blocks(it->second);
        (void)hipGetLastError();
        if (e != hipSuccess) return hip_fail(e, "hipStreamEndCapture");
        if (e2 != hipSuccess) return hip_fail(e2, "hipGraphInstantiate");
        return fail(LQ_ERR_VALUE, "unknown graph id %d", graph_id);
    }
    it->second.graph = graph;
    it->second.exec = exec;
    return LQ_OK;
}

extern "C" int lq_graph_launch(int graph_id, lq_stream stream) {
    hipGraphExec_t exec = nullptr;
    {
        std::lock_guard<std::recursive_mutex> lock(g_rt_mutex);
        auto it = g_graphs.find(graph_id);
        LQ_REQUIRE(it != g_graphs.end() && it->second.exec, LQ_ERR_VALUE, "graph id %d has no executable", graph_id);
        exec = it->second.exec;
    }
    LQ_HIP(hipGraphLaunch(exec, as_stream(stream)));
    return LQ_OK;
}

extern "C" int lq_graph_destroy(int graph_id) {
    std::lock_guard<std::recursive_mutex> lock(g_rt_mutex);
    auto it = g_graphs.find(graph_id);
    if (it == g_graphs.end()) return LQ_OK;
    if (t_capturing_graph == graph_id) t_capturing_graph = 0;
    if (it->second.capturing) {  // destroyed without an end (by whichever thread): the capture is abandoned
        it->second.capturing = false;
        --g_captures_in_progress;
    }
    hipError_t e = hipSuccess;
    if (it->second.exec) e = hipGraphExecDestroy(it->second.exec);
    if (it->second.graph) (void)hipGraphDestroy(it->second.graph);
    unpin_graph_blocks(it->second);
    g_graphs.erase(it);
    drain_retired();
    if (e != hipSuccess) return hip_fail(e, "hipGraphExecDestroy");
    return LQ_OK;
}

int lq_h2d(void* dst, const void* src, size_t nbytes, lq_stream stream) {
    if (nbytes == 0) return LQ_OK;
    LQ_REQUIRE(dst && src, LQ_ERR_VALUE, "NULL pointer in h2d");
    LQ_HIP(hipMemcpyAsync(dst, src, nbytes, hipMemcpyHostToDevice, as_stream(stream)));
    LQ_HIP(hipStreamSynchronize(as_stream(stream)));  // pageable source may be reused at once
    return LQ_OK;
}

int lq_d2h(void* dst, const void* src, size_t nbytes, lq_stream stream) {
    if (nbytes == 0) return LQ_OK;
    LQ_REQUIRE(dst && src, LQ_ERR_VALUE, "NULL pointer in d2h");
    LQ_HIP(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToHost, as_stream(stream)));
    LQ_HIP(hipStreamSynchronize(as_stream(stream)));
    return LQ_OK;
}

int lq_d2d(void* dst, const void* src, size_t nbytes, lq_stream stream) {
    if (nbytes == 0) return LQ_OK;
    LQ_REQUIRE(dst && src, LQ_ERR_VALUE, "NULL pointer in d2d");
    LQ_HIP(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToDevice, as_stream(stream)));
    return LQ_OK;
}

int lq_d2d_rows(void* dst, size_t dst_pitch, const void* src, size_t src_pitch, size_t row_bytes, size_t rows,
                lq_stream stream) {
    if (row_bytes == 0 || rows == 0) return LQ_OK;
    LQ_REQUIRE(dst && src, LQ_ERR_VALUE, "NULL pointer in d2d_rows");
    LQ_REQUIRE(dst_pitch >= row_bytes && src_pitch >= row_bytes, LQ_ERR_SHAPE, "d2d_rows: pitch smaller than a row");
    LQ_HIP(hipMemcpy2DAsync(dst, dst_pitch, src, src_pitch, row_bytes, rows, hipMemcpyDeviceToDevice,
                            as_stream(stream)));
    return LQ_OK;
}

int lq_sync(lq_stream stream) {
    LQ_HIP(hipStreamSynchronize(as_stream(stream)));
    return LQ_OK;
}

int lq_stream_create(lq_stream* stream) {
    LQ_REQUIRE(stream, LQ_ERR_VALUE, "stream is NULL");
    hipStream_t s;
    LQ_HIP(hipStreamCreate(&s));  // default priority only
    *stream = s;
    return LQ_OK;
}

int lq_stream_create_nonblocking(lq_stream* stream) {
    LQ_REQUIRE(stream, LQ_ERR_VALUE, "stream is NULL");
    hipStream_t s;
    LQ_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));  // default priority
    *stream = s;
    return LQ_OK;
}

int lq_stream_destroy(lq_stream stream) {
    if (!stream) return LQ_OK;
    {
        // the stream's scratch goes with it (retired: a graph captured on it may still use it)
        std::lock_guard<std::recursive_mutex> lock(g_rt_mutex);
        for (auto it = g_bufs.begin(); it != g_bufs.end();) {
            if (it->first.stream == as_stream(stream)) {
                if (it->second.ptr) g_retired.push_back(it->second.ptr);
                it = g_bufs.erase(it);
            } else {
                ++it;
            }
        }
    }
    LQ_HIP(hipStreamDestroy(as_stream(stream)));
    std::lock_guard<std::recursive_mutex> lock(g_rt_mutex);
    drain_retired();
    return LQ_OK;
}

int lq_event_create(lq_event* ev) {
    LQ_REQUIRE(ev, LQ_ERR_VALUE, "ev is NULL");
    hipEvent_t e;
    LQ_HIP(hipEventCreate(&e));
    *ev = e;
    return LQ_OK;
}

int lq_event_destroy(lq_event ev) {
    if (ev) LQ_HIP(hipEventDestroy(reinterpret_cast<hipEvent_t>(ev)));
    return LQ_OK;
}

int lq_event_record(lq_event ev, lq_stream stream) {
    LQ_HIP(hipEventRecord(reinterpret_cast<hipEvent_t>(ev), as_stream(stream)));
    return LQ_OK;
}

int lq_stream_wait_event(lq_stream stream, lq_event ev) {
    LQ_REQUIRE(ev, LQ_ERR_VALUE, "stream_wait_event: event is NULL");
    LQ_HIP(hipStreamWaitEvent(as_stream(stream), reinterpret_cast<hipEvent_t>(ev), 0));
    return LQ_OK;
}

int lq_event_sync(lq_event ev) {
    LQ_HIP(hipEventSynchronize(reinterpret_cast<hipEvent_t>(ev)));
    return LQ_OK;
}

int lq_event_elapsed_ms(lq_event start, lq_event stop, float* ms) {
    LQ_REQUIRE(ms, LQ_ERR_VALUE, "ms is NULL");
    LQ_HIP(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start),
                               reinterpret_cast<hipEvent_t>(stop)));
    return LQ_OK;
}

// ------------------------------------------------------------------ op registry
namespace {
struct OpSchema {
    const char* name;
    int version;
    int deterministic;
};
// Integer accumulation is order-independent, so every op here is
// deterministic, the split-K GEMM included.
const OpSchema kOps[] = {
    {"minmax", 1, 1},        {"calc_qparams", 1, 1}, {"quantize", 1, 1},
    {"dequantize", 1, 1},    {"fake_quantize", 1, 1}, {"rowsum_i8", 1, 1},
    {"qlinear_i8", 1, 1},    {"relu", 1, 1},          {"minmax_fold", 1, 1},
    {"add_requant_i8", 1, 1}, {"qconv2d_i8", 1, 1},    {"maxpool2d_nhwc_i8", 1, 1},
    {"global_avgpool_nhwc_i8", 1, 1}, {"qlinear_w8a32", 1, 1},
};
}  // namespace

int lq_op_count(void) { return int(sizeof kOps / sizeof kOps[0]); }

int lq_op_info(int index, const char** name, int* version, int* deterministic) {
    LQ_REQUIRE(index >= 0 && index < lq_op_count(), LQ_ERR_VALUE, "op index %d out of range", index);
    if (name) *name = kOps[index].name;
    if (version) *version = kOps[index].version;
    if (deterministic) *deterministic = kOps[index].deterministic;
    return LQ_OK;
}

}  // extern "C"

// ------------------------------------------------------------------ fills / copy
namespace {

__device__ inline uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

// Two normals per counter (Box-Muller).  Quality is that of a benchmark
// input generator, nothing more.
__global__ void fill_normal_kernel(float* x, size_t n, uint64_t seed, float outlier_prob,
                                   float outlier_gain) {
    size_t pair = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    size_t stride = size_t(gridDim.x) * blockDim.x;
    for (; pair * 2 < n; pair += stride) {
        uint64_t r = splitmix64(seed ^ (pair * 0xD1342543DE82EF95ull));
        uint64_t r2 = splitmix64(r);
        float u1 = (float((r >> 40) + 1)) * (1.0f / 16777217.0f);
        float u2 = float(r & 0xFFFFFF) * (1.0f / 16777216.0f);
        float rad = sqrtf(-2.0f * logf(u1));
        float s, c;
        sincosf(6.28318530718f * u2, &s, &c);
        float a = rad * c, b = rad * s;
        float p1 = float(r2 >> 40) * (1.0f / 16777216.0f);
        float p2 = float(r2 & 0xFFFFFF) * (1.0f / 16777216.0f);
        if (p1 < outlier_prob) a *= outlier_gain;
        if (p2 < outlier_prob) b *= outlier_gain;
        x[pair * 2] = a;
        if (pair * 2 + 1 < n) x[pair * 2 + 1] = b;
    }
}

__global__ void fill_uniform_i8_kernel(int8_t* x, size_t n, uint64_t seed, int lo, int span) {
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    size_t stride = size_t(gridDim.x) * blockDim.x;
    for (; i < n; i += stride) {
        uint64_t r = splitmix64(seed ^ (i * 0xD1342543DE82EF95ull));
        x[i] = int8_t(lo + int((r >> 33) % uint64_t(span)));
    }
}

typedef int probe_v16i __attribute__((ext_vector_type(16)));
typedef int probe_v4i __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void probe_mfma_i8_kernel(const int8_t* __restrict__ a,
                                                            const int8_t* __restrict__ b, int iters,
                                                            int* __restrict__ sink) {
    probe_v16i acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0;
    probe_v4i ra[8], rb[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        ra[i] = reinterpret_cast<const probe_v4i*>(a)[i * 256 + threadIdx.x];
        rb[i] = reinterpret_cast<const probe_v4i*>(b)[i * 256 + threadIdx.x];
    }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ra[i], rb[(i * 3 + 1) & 7], acc[i], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) s ^= acc[i][j];
    // keeps the accumulators live; one word per block, written by one lane
    if (threadIdx.x == 0) sink[0] = s;
}

// The same probe with the instruction and the walk of the large-GEMM kernel: a wavefront owns
// 4 x 11 tiles of v_mfma_i32_16x16x64_i8, visits them column by column with the row order
// alternating (one operand changes between neighbours), two wavefronts per SIMD.
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void probe_mfma_i8_k64_kernel(
    const int8_t* __restrict__ a, const int8_t* __restrict__ b, int iters, int* __restrict__ sink) {
    probe_v4i acc[4][11];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 11; ++j) acc[i][j] = probe_v4i{0, 0, 0, 0};
    probe_v4i ra[4], rb[11];
#pragma unroll
    for (int i = 0; i < 4; ++i) ra[i] = reinterpret_cast<const probe_v4i*>(a)[i * 256 + threadIdx.x];
#pragma unroll
    for (int j = 0; j < 11; ++j) rb[j] = reinterpret_cast<const probe_v4i*>(b)[j * 256 + threadIdx.x];
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 11; ++j)
#pragma unroll
            for (int ii = 0; ii < 4; ++ii) {
                const int i = (j & 1) ? 3 - ii : ii;
                acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(rb[j], ra[i], acc[i][j], 0, 0, 0);
            }
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 11; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) s ^= acc[i][j][r];
    if (threadIdx.x == 0) sink[0] = s;
}

__global__ void fill_bytes_kernel(uint8_t* x, size_t n, uint8_t v) {
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    size_t stride = size_t(gridDim.x) * blockDim.x;
    for (; i < n; i += stride) x[i] = v;
}

__global__ void copy16_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t n16) {
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    size_t stride = size_t(gridDim.x) * blockDim.x;
    for (; i < n16; i += stride) dst[i] = src[i];
}

inline unsigned blocks_for(size_t work, unsigned per_block, unsigned cap) {
    size_t b = (work + per_block - 1) / per_block;
    if (b < 1) b = 1;
    return unsigned(b > cap ? cap : b);
}

}  // namespace

extern "C" {

int lq_fill_normal(float* x, size_t n, uint64_t seed, float outlier_prob, float outlier_gain,
                   lq_stream stream) {
    if (n == 0) return LQ_OK;
    LQ_REQUIRE(x, LQ_ERR_VALUE, "x is NULL");
    hipLaunchKernelGGL(fill_normal_kernel, dim3(blocks_for((n + 1) / 2, 256, 65536)), dim3(256), 0,
                       as_stream(stream), x, n, seed, outlier_prob, outlier_gain);
    LQ_CHECK_LAUNCH("fill_normal");
    return LQ_OK;
}

int lq_fill_uniform_i8(int8_t* x, size_t n, uint64_t seed, int lo, int hi, lq_stream stream) {
    if (n == 0) return LQ_OK;
    LQ_REQUIRE(x, LQ_ERR_VALUE, "x is NULL");
    LQ_REQUIRE(lo >= -128 && hi <= 127 && lo <= hi, LQ_ERR_VALUE, "bad int8 range [%d,%d]", lo, hi);
    hipLaunchKernelGGL(fill_uniform_i8_kernel, dim3(blocks_for(n, 256, 65536)), dim3(256), 0,
                       as_stream(stream), x, n, seed, lo, hi - lo + 1);
    LQ_CHECK_LAUNCH("fill_uniform_i8");
    return LQ_OK;
}

// Matrix-core rate probe: every wavefront keeps eight 32x32 int32 accumulators
// and issues `iters` rounds of eight v_mfma_i32_32x32x32_i8 whose operands
// rotate over eight register sets taken from `a` and `b`, so operand bits
// toggle between instructions the way they do in a GEMM over that data.  No
// LDS or memory traffic inside the loop: the rate is what the matrix cores
// sustain for these operand statistics under the board's power limit.
int lq_probe_mfma_i8(const int8_t* a, const int8_t* b, size_t nbytes, int iters, int* sink, double* ops,
                     lq_stream stream) {
    LQ_REQUIRE(a && b && sink && ops, LQ_ERR_VALUE, "probe_mfma_i8: NULL pointer");
    LQ_REQUIRE(iters > 0, LQ_ERR_VALUE, "probe_mfma_i8: iters must be positive");
    LQ_REQUIRE(nbytes >= size_t(256) * 8 * 16, LQ_ERR_SHAPE, "probe_mfma_i8: need at least 32 KiB of operand data");
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(a) % 16 == 0 && reinterpret_cast<uintptr_t>(b) % 16 == 0, LQ_ERR_VALUE,
               "probe_mfma_i8: operands must be 16-byte aligned");
    int dev = 0, cus = 0;
    LQ_HIP(hipGetDevice(&dev));
    LQ_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int blocks = 2 * cus;  // two wavefronts per SIMD
    hipLaunchKernelGGL(probe_mfma_i8_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), a, b, iters, sink);
    LQ_CHECK_LAUNCH("probe_mfma_i8");
    *ops = double(blocks) * 4.0 * double(iters) * 8.0 * (2.0 * 32 * 32 * 32);
    return LQ_OK;
}

int lq_probe_mfma_i8_k64(const int8_t* a, const int8_t* b, size_t nbytes, int iters, int* sink, double* ops,
                         lq_stream stream) {
    LQ_REQUIRE(a && b && sink && ops, LQ_ERR_VALUE, "probe_mfma_i8_k64: NULL pointer");
    LQ_REQUIRE(iters > 0, LQ_ERR_VALUE, "probe_mfma_i8_k64: iters must be positive");
    LQ_REQUIRE(nbytes >= size_t(256) * 11 * 16, LQ_ERR_SHAPE, "probe_mfma_i8_k64: need at least 44 KiB of operand data");
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(a) % 16 == 0 && reinterpret_cast<uintptr_t>(b) % 16 == 0, LQ_ERR_VALUE,
               "probe_mfma_i8_k64: operands must be 16-byte aligned");
    int dev = 0, cus = 0;
    LQ_HIP(hipGetDevice(&dev));
    LQ_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int blocks = 2 * cus;  // two wavefronts per SIMD
    hipLaunchKernelGGL(probe_mfma_i8_k64_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), a, b, iters, sink);
    LQ_CHECK_LAUNCH("probe_mfma_i8_k64");
    *ops = double(blocks) * 4.0 * double(iters) * 44.0 * (2.0 * 16 * 16 * 64);
    return LQ_OK;
}

// A fill kernel rather than hipMemsetAsync so that callers may capture it in
// a HIP graph.
int lq_fill_bytes(void* dst, int value, size_t nbytes, lq_stream stream) {
    if (nbytes == 0) return LQ_OK;
    LQ_REQUIRE(dst, LQ_ERR_VALUE, "dst is NULL");
    hipLaunchKernelGGL(fill_bytes_kernel, dim3(blocks_for(nbytes, 256, 65536)), dim3(256), 0,
                       as_stream(stream), static_cast<uint8_t*>(dst), nbytes, uint8_t(value));
    LQ_CHECK_LAUNCH("fill_bytes");
    return LQ_OK;
}

int lq_copy_kernel(void* dst, const void* src, size_t nbytes, lq_stream stream) {
    LQ_REQUIRE(dst && src, LQ_ERR_VALUE, "NULL pointer");
    LQ_REQUIRE(nbytes % 16 == 0 && aligned16(dst) && aligned16(src), LQ_ERR_VALUE,
               "copy kernel needs 16-byte aligned pointers and size");
    if (nbytes == 0) return LQ_OK;
    hipLaunchKernelGGL(copy16_kernel, dim3(blocks_for(nbytes / 16, 256, 1 << 20)), dim3(256), 0,
                       as_stream(stream), static_cast<uint4*>(dst), static_cast<const uint4*>(src),
                       nbytes / 16);
    LQ_CHECK_LAUNCH("copy16");
    return LQ_OK;
}

}  // extern "C"
