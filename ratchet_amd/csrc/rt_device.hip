// Device, storage and timing entry points of the C ABI: hipMalloc'd storage and one in-order stream take the place
// of ratchet-core's wgpu device, buffer pool and queue (gpu/device.rs, gpu/pools/buffer_pool.rs,
// storage/gpu_buffer.rs in crates/ratchet-core/src).
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <unordered_map>

#include "rt_internal.h"

struct rt_graph {
    hipGraph_t graph;
    hipGraphExec_t exec;
    int ordinal;
};

struct rt_parked {
    void* ptr;
    uint64_t pass;                                  // the pass (rt_pool_begin_pass count) during which the block was freed
};
struct rt_pool {
    std::mutex mu;
    std::multimap<size_t, rt_parked> parked;        // block size -> block, free for reuse
    uint64_t pass = 0;
    std::unordered_map<void*, size_t> live;         // blocks handed out by rt_malloc
    size_t parked_bytes = 0;
    size_t live_bytes = 0, peak_live_bytes = 0;     // handed out now / the most that was handed out at once since the last reset
    uint64_t hits = 0, misses = 0;
};

static thread_local char g_err[512] = "";

int rt_fail(int status, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return status;
}

int rt_fail_hip(hipError_t e, const char* what) {
    snprintf(g_err, sizeof(g_err), "%s: %s (%s)", what, hipGetErrorString(e), hipGetErrorName(e));
    (void)hipGetLastError();   // clear the sticky error so the next call reports its own
    return -(int)e;
}

int rt_enter(rt_device* dev) {
    if (!dev) return rt_fail(RT_ERR_NULL_DEVICE, "rt_device is NULL");
    hipError_t e = hipSetDevice(dev->ordinal);
    if (e != hipSuccess) return rt_fail_hip(e, "hipSetDevice");
    return RT_OK;
}

// bytes [0, head) and the tail after the last whole 16-byte vector are cleared bytewise by block 0
__global__ void __launch_bounds__(256) zero_bytes_kernel(unsigned char* p, size_t head, size_t nvec, size_t bytes) {
    uint4* v = reinterpret_cast<uint4*>(p + head);
    const size_t base = (size_t)blockIdx.x * (256 * 4) + threadIdx.x;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const size_t i = base + (size_t)k * 256;
        if (i < nvec) v[i] = make_uint4(0, 0, 0, 0);
    }
    if (blockIdx.x == 0) {
        const size_t tail_start = head + nvec * 16;
        for (size_t i = threadIdx.x; i < head; i += 256) p[i] = 0;
        for (size_t i = tail_start + threadIdx.x; i < bytes; i += 256) p[i] = 0;
    }
}

extern "C" {

const char* rt_last_error(void) { return g_err; }

int rt_debug_hip_status(int hip_error, const char* what) {
    if (hip_error == 0) return RT_OK;
    return rt_fail_hip((hipError_t)hip_error, what ? what : "injected");
}

int rt_debug_softmax_pace(rt_device* dev, uint32_t ticks) {
    if (!dev) return rt_fail(RT_ERR_NULL_DEVICE, "rt_device is NULL");
    RT_REQUIRE(ticks < (1u << 30), RT_ERR_ARG, "rt_debug_softmax_pace: %u ticks out of range", ticks);
    dev->debug_softmax_pace = ticks;
    return RT_OK;
}

const char* rt_status_name(int status) {
    switch (status) {
        case RT_OK: return "RT_OK";
        case RT_ERR_NULL_POINTER: return "RT_ERR_NULL_POINTER";
        case RT_ERR_DTYPE: return "RT_ERR_DTYPE";
        case RT_ERR_OP: return "RT_ERR_OP";
        case RT_ERR_SHAPE: return "RT_ERR_SHAPE";
        case RT_ERR_PERM: return "RT_ERR_PERM";
        case RT_ERR_SIZE: return "RT_ERR_SIZE";
        case RT_ERR_ARG: return "RT_ERR_ARG";
        case RT_ERR_NULL_DEVICE: return "RT_ERR_NULL_DEVICE";
        case RT_ERR_ALIGN: return "RT_ERR_ALIGN";
        case RT_ERR_CAPTURE: return "RT_ERR_CAPTURE";
        default: return status < 0 ? "HIP_ERROR" : "RT_ERR_UNKNOWN";
    }
}

int rt_device_count(int* out) {
    RT_REQUIRE(out, RT_ERR_NULL_POINTER, "rt_device_count: out is NULL");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        *out = 0;
        return rt_fail_hip(e, "hipGetDeviceCount");
    }
    *out = n;
    return RT_OK;
}

int rt_device_create(int ordinal, rt_device** out) {
    RT_REQUIRE(out, RT_ERR_NULL_POINTER, "rt_device_create: out is NULL");
    *out = nullptr;
    RT_REQUIRE(ordinal >= 0, RT_ERR_ARG, "rt_device_create: negative ordinal %d", ordinal);
    int n = 0;
    RT_HIP(hipGetDeviceCount(&n));
    RT_REQUIRE(ordinal < n, RT_ERR_ARG, "rt_device_create: ordinal %d but %d device(s) visible", ordinal, n);
    RT_HIP(hipSetDevice(ordinal));
    hipDeviceProp_t prop;
    RT_HIP(hipGetDeviceProperties(&prop, ordinal));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return rt_fail(RT_ERR_ARG, "rt_device_create: device %d is %s; this library is built for gfx950 only", ordinal,
                       prop.gcnArchName);
    rt_device* dev = new rt_device();
    memset(dev, 0, sizeof(*dev));
    dev->pool = new rt_pool();
    dev->ordinal = ordinal;
    dev->num_cus = prop.multiProcessorCount;
    {
        int khz = 0;
        if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, ordinal) != hipSuccess) (void)hipGetLastError();
        dev->wall_clock_hz = khz > 0 ? khz * 1e3 : 1e8;
        dev->debug_softmax_pace = 0;
    }
    hipError_t e = hipStreamCreateWithFlags(&dev->stream, hipStreamNonBlocking);   // default priority
    if (e != hipSuccess) {
        delete dev->pool;
        delete dev;
        return rt_fail_hip(e, "hipStreamCreateWithFlags");
    }
    dev->gn_scratch_bytes = 1u << 20;
    e = hipMalloc((void**)&dev->gn_scratch, dev->gn_scratch_bytes);
    if (e != hipSuccess) {
        (void)hipStreamDestroy(dev->stream);
        delete dev->pool;
        delete dev;
        return rt_fail_hip(e, "hipMalloc(scratch)");
    }
    e = hipMalloc((void**)&dev->sm_row_sums, RT_SM_ROW_SUMS * sizeof(uint16_t) + (RT_SM_TILES_HEAD + RT_SM_MASK_TILES) * sizeof(uint32_t));
    if (e == hipSuccess) {
        dev->sm_mask_tiles = reinterpret_cast<uint32_t*>(dev->sm_row_sums + RT_SM_ROW_SUMS);
        e = hipMemset(dev->sm_mask_tiles, 0xff, RT_SM_TILES_HEAD * sizeof(uint32_t));
        if (e != hipSuccess) (void)hipFree(dev->sm_row_sums);
    }
    if (e != hipSuccess) {
        (void)hipFree(dev->gn_scratch);
        (void)hipStreamDestroy(dev->stream);
        delete dev->pool;
        delete dev;
        return rt_fail_hip(e, "hipMalloc(row sums)");
    }
    int rc = rt_norm_device_init(dev);
    if (rc) {
        (void)hipFree(dev->sm_row_sums);
        (void)hipFree(dev->gn_scratch);
        (void)hipStreamDestroy(dev->stream);
        delete dev->pool;
        delete dev;
        return rc;
    }
    *out = dev;
    return RT_OK;
}

int rt_device_destroy(rt_device* dev) {
    int rc = rt_enter(dev);
    if (rc) return rc;
    RT_NO_CAPTURE(dev, "rt_device_destroy");
    (void)hipStreamSynchronize(dev->stream);
    for (int t = 0; t < 2; t++)
        for (int i = 0; i < RT_UNARY_COUNT; i++)
        {
            if (dev->unary_lut[t][i]) (void)hipFree(dev->unary_lut[t][i]);
            if (dev->unary_lut_via32[t][i]) (void)hipFree(dev->unary_lut_via32[t][i]);
        }
    if (dev->gn_scratch) (void)hipFree(dev->gn_scratch);
    if (dev->sm_row_sums) (void)hipFree(dev->sm_row_sums);
    // buffers the caller never returned are released with the device, like the parked ones
    for (auto& kv : dev->pool->parked) (void)hipFree(kv.second.ptr);
    for (auto& kv : dev->pool->live) (void)hipFree(kv.first);
    delete dev->pool;
    hipError_t e = hipStreamDestroy(dev->stream);
    delete dev;
    if (e != hipSuccess) return rt_fail_hip(e, "hipStreamDestroy");
    return RT_OK;
}

int rt_sync(rt_device* dev) {
    int rc = rt_enter(dev);
    if (rc) return rc;
    RT_NO_CAPTURE(dev, "rt_sync");
    RT_HIP(hipStreamSynchronize(dev->stream));
    return RT_OK;
}

// Storage pool.  The reference keeps freed GPU buffers in a pool keyed by size and hands them out again
// (crates/ratchet-core/src/gpu/pools/buffer_pool.rs:60-112) because creating a buffer per op per step is what costs.
// Here: rt_free parks the block, rt_malloc takes the smallest parked block that fits without wasting more than a
// quarter of it.  Every kernel and copy of a device runs on that device's one stream, so a block handed out again is
// only touched by work queued after the work of its previous owner: no synchronisation is needed on either call.
// hipMalloc / hipFree (which synchronise the device) happen only on a pool miss, in rt_pool_trim and at destroy.
static size_t pool_round(size_t bytes) {
    // the reference rounds sizes up to 4 bytes and never allocates less than 16 (buffer_pool.rs:82-93); blocks are
    // further rounded so that near-equal requests share a size: 512 B steps up to 1 MiB, 1/16 of the size above
    size_t sz = (bytes + 3) & ~(size_t)3;
    if (sz < 16) sz = 16;
    if (sz <= (1u << 20)) return (sz + 511) & ~(size_t)511;
    size_t step = 1;
    while (step * 32 <= sz) step <<= 1;                          // step = 2^floor(log2(sz)) / 16
    return (sz + step - 1) / step * step;
}

int rt_malloc(rt_device* dev, size_t bytes, void** dptr) {
    RT_REQUIRE(dptr, RT_ERR_NULL_POINTER, "rt_malloc: dptr is NULL");
    *dptr = nullptr;
    int rc = rt_enter(dev);
    if (rc) return rc;
    const size_t sz = pool_round(bytes);
    rt_pool* pool = dev->pool;
    std::lock_guard<std::mutex> lock(pool->mu);
    auto it = pool->parked.lower_bound(sz);
    if (it != pool->parked.end() && it->first <= sz + sz / 4) {
        *dptr = it->second.ptr;
        pool->live.emplace(it->second.ptr, it->first);
        pool->live_bytes += it->first;
        if (pool->live_bytes > pool->peak_live_bytes) pool->peak_live_bytes = pool->live_bytes;
        pool->parked_bytes -= it->first;
        pool->parked.erase(it);
        pool->hits++;
        return RT_OK;
    }
    RT_NO_CAPTURE(dev, "rt_malloc of a size the pool holds no block for");
    hipError_t e = hipMalloc(dptr, sz);
    if (e == hipErrorOutOfMemory && !pool->parked.empty()) {   // give the parked blocks back and try once more
        (void)hipGetLastError();
        (void)hipStreamSynchronize(dev->stream);
        for (auto& kv : pool->parked) (void)hipFree(kv.second.ptr);
        pool->parked.clear();
        pool->parked_bytes = 0;
        e = hipMalloc(dptr, sz);
    }
    if (e != hipSuccess) {
        *dptr = nullptr;
        return rt_fail_hip(e, "hipMalloc");
    }
    pool->live.emplace(*dptr, sz);
    pool->live_bytes += sz;
    if (pool->live_bytes > pool->peak_live_bytes) pool->peak_live_bytes = pool->live_bytes;
    pool->misses++;
    return RT_OK;
}

int rt_free(rt_device* dev, void* dptr) {
    int rc = rt_enter(dev);
    if (rc) return rc;
    if (!dptr) return RT_OK;
    rt_pool* pool = dev->pool;
    std::lock_guard<std::mutex> lock(pool->mu);
    auto it = pool->live.find(dptr);
    RT_REQUIRE(it != pool->live.end(), RT_ERR_ARG, "rt_free: %p was not allocated by rt_malloc on this device (or was freed twice)", dptr);
    pool->parked.emplace(it->second, rt_parked{dptr, pool->pass});
    pool->parked_bytes += it->second;
    pool->live_bytes -= it->second;
    pool->live.erase(it);
    return RT_OK;
}

int rt_pool_trim(rt_device* dev) {
    int rc = rt_enter(dev);
    if (rc) return rc;
    RT_NO_CAPTURE(dev, "rt_pool_trim");
    RT_HIP(hipStreamSynchronize(dev->stream));                  // queued work may still use a parked block
    rt_pool* pool = dev->pool;
    std::lock_guard<std::mutex> lock(pool->mu);
    hipError_t first = hipSuccess;
    for (auto& kv : pool->parked) {
        hipError_t e = hipFree(kv.second.ptr);
        if (e != hipSuccess && first == hipSuccess) first = e;
    }
    pool->parked.clear();
    pool->parked_bytes = 0;
    if (first != hipSuccess) return rt_fail_hip(first, "hipFree");
    return RT_OK;
}

// The reference's pool ages its unused buffers by passes (gpu/pools/dynamic_resource_pool.rs:140-190, called at the top of
// every resolve: tensor.rs:800, gpu/device.rs:275-277): a buffer released during pass p can be reclaimed during pass
// p + 1 and is destroyed at the start of pass p + 2 if nobody did.  The same here: a block parked before the previous
// call of this function, and still parked, goes back to the driver.  A program that repeats its passes reuses every
// block each time and never gets here with anything to free, so the steady state stays free of hipFree (and of the wait
// for the stream that has to precede it); one whose sizes drift no longer grows the parked set without bound.  While a
// device is capturing nothing is freed: the blocks wait for the first pass that begins outside a capture.
int rt_pool_begin_pass(rt_device* dev) {
    int rc = rt_enter(dev);
    if (rc) return rc;
    rt_pool* pool = dev->pool;
    std::lock_guard<std::mutex> lock(pool->mu);
    const uint64_t now = ++pool->pass;                          // blocks freed from here on carry `now`
    if (dev->capturing) return RT_OK;
    bool stale = false;
    for (auto& kv : pool->parked) stale = stale || kv.second.pass + 2 <= now;
    if (!stale) return RT_OK;
    RT_HIP(hipStreamSynchronize(dev->stream));                  // queued work may still use a parked block
    hipError_t first = hipSuccess;
    for (auto it = pool->parked.begin(); it != pool->parked.end();) {
        if (it->second.pass + 2 <= now) {
            hipError_t e = hipFree(it->second.ptr);
            if (e != hipSuccess && first == hipSuccess) first = e;
            pool->parked_bytes -= it->first;
            it = pool->parked.erase(it);
        } else {
            ++it;
        }
    }
    if (first != hipSuccess) return rt_fail_hip(first, "hipFree");
    return RT_OK;
}

int rt_pool_stats(rt_device* dev, uint64_t* live_bytes, uint64_t* parked_bytes, uint64_t* hits, uint64_t* misses) {
    RT_REQUIRE(dev, RT_ERR_NULL_DEVICE, "rt_device is NULL");
    rt_pool* pool = dev->pool;
    std::lock_guard<std::mutex> lock(pool->mu);
    uint64_t live = 0;
    for (auto& kv : pool->live) live += kv.second;
    if (live_bytes) *live_bytes = live;
    if (parked_bytes) *parked_bytes = pool->parked_bytes;
    if (hits) *hits = pool->hits;
    if (misses) *misses = pool->misses;
    return RT_OK;
}

int rt_pool_peak(rt_device* dev, uint64_t* peak_live_bytes, int reset) {
    RT_REQUIRE(dev, RT_ERR_NULL_DEVICE, "rt_device is NULL");
    rt_pool* pool = dev->pool;
    std::lock_guard<std::mutex> lock(pool->mu);
    if (peak_live_bytes) *peak_live_bytes = pool->peak_live_bytes;
    if (reset) pool->peak_live_bytes = pool->live_bytes;
    return RT_OK;
}

int rt_memset0(rt_device* dev, void* dptr, size_t bytes) {
    RT_REQUIRE(dptr || bytes == 0, RT_ERR_NULL_POINTER, "rt_memset0: dptr is NULL");
    int rc = rt_enter(dev);
    if (rc) return rc;
    if (bytes == 0) return RT_OK;
    // a fill kernel rather than hipMemsetAsync, so that a caller may capture this call in a HIP graph
    const uintptr_t addr = reinterpret_cast<uintptr_t>(dptr);
    const size_t head = (size_t)((16 - (addr & 15)) & 15) < bytes ? (size_t)((16 - (addr & 15)) & 15) : bytes;
    const size_t nvec = (bytes - head) / 16;
    const size_t per_block = 256 * 4;
    const size_t blocks = nvec ? (nvec + per_block - 1) / per_block : 1;
    RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "rt_memset0: %zu bytes is too large", bytes);
    hipLaunchKernelGGL(zero_bytes_kernel, dim3((unsigned)blocks), dim3(256), 0, dev->stream, (unsigned char*)dptr, head,
                       nvec, bytes);
    RT_CHECK_LAUNCH("zero_bytes_kernel");
    return RT_OK;
}

int rt_h2d(rt_device* dev, void* dptr, const void* host, size_t bytes) {
    RT_REQUIRE((dptr && host) || bytes == 0, RT_ERR_NULL_POINTER, "rt_h2d: NULL pointer");
    int rc = rt_enter(dev);
    if (rc) return rc;
    if (bytes == 0) return RT_OK;
    RT_NO_CAPTURE(dev, "rt_h2d");
    RT_HIP(hipMemcpyAsync(dptr, host, bytes, hipMemcpyHostToDevice, dev->stream));
    RT_HIP(hipStreamSynchronize(dev->stream));
    return RT_OK;
}

int rt_d2h(rt_device* dev, void* host, const void* dptr, size_t bytes) {
    RT_REQUIRE((dptr && host) || bytes == 0, RT_ERR_NULL_POINTER, "rt_d2h: NULL pointer");
    int rc = rt_enter(dev);
    if (rc) return rc;
    if (bytes == 0) return RT_OK;
    RT_NO_CAPTURE(dev, "rt_d2h");
    RT_HIP(hipMemcpyAsync(host, dptr, bytes, hipMemcpyDeviceToHost, dev->stream));
    RT_HIP(hipStreamSynchronize(dev->stream));
    return RT_OK;
}

int rt_d2d(rt_device* dev, void* dst, const void* src, size_t bytes) {
    RT_REQUIRE((dst && src) || bytes == 0, RT_ERR_NULL_POINTER, "rt_d2d: NULL pointer");
    int rc = rt_enter(dev);
    if (rc) return rc;
    if (bytes == 0) return RT_OK;
    RT_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, dev->stream));
    return RT_OK;
}

int rt_capture_begin(rt_device* dev) {
    int rc = rt_enter(dev);
    if (rc) return rc;
    RT_REQUIRE(!dev->capturing, RT_ERR_CAPTURE, "rt_capture_begin: the device is already capturing");
    // thread-local mode: only this thread's calls on this stream are checked, other threads and devices carry on
    RT_HIP(hipStreamBeginCapture(dev->stream, hipStreamCaptureModeThreadLocal));
    dev->capturing = 1;
    return RT_OK;
}

int rt_capture_end(rt_device* dev, rt_graph** out) {
    RT_REQUIRE(out, RT_ERR_NULL_POINTER, "rt_capture_end: out is NULL");
    *out = nullptr;
    int rc = rt_enter(dev);
    if (rc) return rc;
    RT_REQUIRE(dev->capturing, RT_ERR_CAPTURE, "rt_capture_end: the device is not capturing");
    dev->capturing = 0;
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(dev->stream, &graph);
    if (e != hipSuccess || !graph) return e != hipSuccess ? rt_fail_hip(e, "hipStreamEndCapture") : rt_fail(RT_ERR_CAPTURE, "rt_capture_end: empty capture");
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(graph);
        return rt_fail_hip(e, "hipGraphInstantiate");
    }
    rt_graph* g = new rt_graph();
    g->graph = graph;
    g->exec = exec;
    g->ordinal = dev->ordinal;
    *out = g;
    return RT_OK;
}

int rt_graph_launch(rt_device* dev, rt_graph* graph) {
    RT_REQUIRE(graph, RT_ERR_NULL_POINTER, "rt_graph_launch: graph is NULL");
    int rc = rt_enter(dev);
    if (rc) return rc;
    RT_NO_CAPTURE(dev, "rt_graph_launch");
    RT_REQUIRE(graph->ordinal == dev->ordinal, RT_ERR_ARG, "rt_graph_launch: the graph was captured on device %d", graph->ordinal);
    RT_HIP(hipGraphLaunch(graph->exec, dev->stream));
    return RT_OK;
}

int rt_graph_destroy(rt_graph* graph) {
    if (!graph) return RT_OK;
    (void)hipSetDevice(graph->ordinal);
    hipError_t e1 = hipGraphExecDestroy(graph->exec);
    hipError_t e2 = hipGraphDestroy(graph->graph);
    delete graph;
    if (e1 != hipSuccess) return rt_fail_hip(e1, "hipGraphExecDestroy");
    if (e2 != hipSuccess) return rt_fail_hip(e2, "hipGraphDestroy");
    return RT_OK;
}

int rt_event_create(rt_device* dev, rt_event** out) {
    RT_REQUIRE(out, RT_ERR_NULL_POINTER, "rt_event_create: out is NULL");
    *out = nullptr;
    int rc = rt_enter(dev);
    if (rc) return rc;
    rt_event* ev = new rt_event();
    ev->ordinal = dev->ordinal;
    hipError_t e = hipEventCreate(&ev->ev);
    if (e != hipSuccess) {
        delete ev;
        return rt_fail_hip(e, "hipEventCreate");
    }
    *out = ev;
    return RT_OK;
}

int rt_event_destroy(rt_event* ev) {
    RT_REQUIRE(ev, RT_ERR_NULL_POINTER, "rt_event_destroy: event is NULL");
    (void)hipSetDevice(ev->ordinal);
    hipError_t e = hipEventDestroy(ev->ev);
    delete ev;
    if (e != hipSuccess) return rt_fail_hip(e, "hipEventDestroy");
    return RT_OK;
}

int rt_event_record(rt_device* dev, rt_event* ev) {
    RT_REQUIRE(ev, RT_ERR_NULL_POINTER, "rt_event_record: event is NULL");
    int rc = rt_enter(dev);
    if (rc) return rc;
    RT_NO_CAPTURE(dev, "rt_event_record");
    RT_HIP(hipEventRecord(ev->ev, dev->stream));
    return RT_OK;
}

int rt_event_elapsed_ms(rt_event* start, rt_event* stop, float* ms) {
    RT_REQUIRE(start && stop && ms, RT_ERR_NULL_POINTER, "rt_event_elapsed_ms: NULL argument");
    (void)hipSetDevice(stop->ordinal);
    RT_HIP(hipEventSynchronize(stop->ev));
    RT_HIP(hipEventElapsedTime(ms, start->ev, stop->ev));
    return RT_OK;
}

}  // extern "C"
