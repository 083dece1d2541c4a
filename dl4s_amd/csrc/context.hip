// Context, pooled allocator, copies and the stream timer of libdl4s_hip.so.
#include "common.h"

#include <algorithm>
#include <functional>

#include <cstdlib>
#include <cstring>

namespace dl4s {

static thread_local char g_err[512] = "";

int set_error(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_error(hipError_t e, const char *what) {
    snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(e));
    (void)hipGetLastError();  // clear the sticky flag so that the next call reports its own failure
    return e == hipErrorOutOfMemory ? DL4S_HIP_EOOM : DL4S_HIP_EHIP;
}

// Allocation sizes are rounded so that freed blocks are reusable: 512 B granules up to 1 MiB,
// 2 MiB granules above.
static size_t round_size(size_t bytes) {
    if (bytes == 0) bytes = 1;
    const size_t small = 512, large = size_t(2) << 20;
    if (bytes <= (size_t(1) << 20)) return (bytes + small - 1) / small * small;
    return (bytes + large - 1) / large * large;
}

int ensure_scratch(dl4s_hip_ctx *ctx, size_t bytes) {
    std::lock_guard<std::mutex> g(ctx->mu);
    if (bytes <= ctx->scratch_bytes) return DL4S_HIP_OK;
    DL4S_REQUIRE(!ctx->capturing, DL4S_HIP_EUNSUPPORTED,
                 "a call recorded into a graph needs %zu bytes of library scratch and %zu are there: run the same calls "
                 "once before recording them", bytes, ctx->scratch_bytes);
    // the old block may still be read by enqueued kernels: wait before releasing it
    if (ctx->scratch) {
        DL4S_HIP_TRY(hipStreamSynchronize(ctx->stream));
        DL4S_HIP_TRY(hipFree(ctx->scratch));
        ctx->scratch = nullptr;
        ctx->scratch_bytes = 0;
        // graphs recorded so far hold the freed address: they are refused from here on, whether or not the new block comes
        ++ctx->scratch_generation;
    }
    size_t want = round_size(bytes);
    DL4S_HIP_TRY(hipMalloc(&ctx->scratch, want));
    ctx->scratch_bytes = want;
    ++ctx->scratch_generation;
    return DL4S_HIP_OK;
}

}  // namespace dl4s

using namespace dl4s;

extern "C" {

const char *dl4s_hip_last_error(void) { return g_err; }

int dl4s_hip_create(int device_ordinal, dl4s_hip_ctx **out_ctx) {
    DL4S_REQUIRE(out_ctx, DL4S_HIP_EINVALID_ARG, "dl4s_hip_create: out_ctx is NULL");
    *out_ctx = nullptr;
    int n = 0;
    DL4S_HIP_TRY(hipGetDeviceCount(&n));
    DL4S_REQUIRE(device_ordinal >= 0 && device_ordinal < n, DL4S_HIP_EINVALID_ARG,
                 "dl4s_hip_create: device %d not in [0,%d)", device_ordinal, n);
    DL4S_HIP_TRY(hipSetDevice(device_ordinal));
    hipDeviceProp_t prop;
    DL4S_HIP_TRY(hipGetDeviceProperties(&prop, device_ordinal));
    DL4S_REQUIRE(strncmp(prop.gcnArchName, "gfx950", 6) == 0, DL4S_HIP_EUNSUPPORTED,
                 "dl4s_hip_create: device %d is %s; this library holds gfx950 code only", device_ordinal,
                 prop.gcnArchName);
    dl4s_hip_ctx *c = new (std::nothrow) dl4s_hip_ctx();
    DL4S_REQUIRE(c, DL4S_HIP_EOOM, "dl4s_hip_create: host allocation failed");
    c->device = device_ordinal;
    c->cu_count = prop.multiProcessorCount;
    c->clock_khz = prop.clockRate;
    // some driver stacks leave the marketing name of the properties empty: ask the other query, then say so
    char queried[128] = "";
    if (!prop.name[0] && hipDeviceGetName(queried, (int)sizeof(queried), device_ordinal) != hipSuccess) queried[0] = 0;
    (void)hipGetLastError();
    if (prop.name[0] || queried[0])
        snprintf(c->name, sizeof(c->name), "%s (%s)", prop.name[0] ? prop.name : queried, prop.gcnArchName);
    else   // name the GPU by what the properties do hold
        snprintf(c->name, sizeof(c->name), "AMD GPU %s, %d CUs, %.2f GHz, %.0f GiB", prop.gcnArchName, prop.multiProcessorCount,
                 prop.clockRate * 1e-6, (double)prop.totalGlobalMem / (double)(1ull << 30));
    hipError_t e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreate(&c->ev_begin);
    if (e == hipSuccess) e = hipEventCreate(&c->ev_end);
    if (e != hipSuccess) {
        if (c->ev_end) (void)hipEventDestroy(c->ev_end);
        if (c->ev_begin) (void)hipEventDestroy(c->ev_begin);
        if (c->stream) (void)hipStreamDestroy(c->stream);
        delete c;
        return hip_error(e, "dl4s_hip_create");
    }
    {
        const int rc = decode_static_scratch_init(c);
        if (rc) {
            decode_static_scratch_release(c);
            (void)hipEventDestroy(c->ev_end);
            (void)hipEventDestroy(c->ev_begin);
            (void)hipStreamDestroy(c->stream);
            delete c;
            return rc;
        }
    }
    *out_ctx = c;
    return DL4S_HIP_OK;
}

int dl4s_hip_destroy(dl4s_hip_ctx *ctx) {
    DL4S_CHECK_CTX(ctx);
    if (ctx->capturing) {   // an open recording is given up
        hipGraph_t recorded = nullptr;
        if (hipStreamEndCapture(ctx->stream, &recorded) == hipSuccess && recorded) (void)hipGraphDestroy(recorded);
        (void)hipGetLastError();
        ctx->capturing = false;
    }
    (void)hipStreamSynchronize(ctx->stream);
    decode_static_scratch_release(ctx);
    for (auto &b : ctx->held_by_recording) (void)hipFree(b.first);
    for (auto &kv : ctx->pool)
        for (void *p : kv.second) (void)hipFree(p);
    for (auto &kv : ctx->live) (void)hipFree(reinterpret_cast<void *>(kv.first));
    if (ctx->scratch) (void)hipFree(ctx->scratch);
    (void)hipEventDestroy(ctx->ev_begin);
    (void)hipEventDestroy(ctx->ev_end);
    (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return DL4S_HIP_OK;
}

int dl4s_hip_sync(dl4s_hip_ctx *ctx) {
    DL4S_CHECK_CTX(ctx);
    DL4S_NOT_WHILE_CAPTURING(ctx);
    DL4S_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return DL4S_HIP_OK;
}

int dl4s_hip_device_info(dl4s_hip_ctx *ctx, int *out_cu_count, int *out_clock_khz, char *name_buf, size_t name_len) {
    DL4S_CHECK_CTX(ctx);
    if (out_cu_count) *out_cu_count = ctx->cu_count;
    if (out_clock_khz) *out_clock_khz = ctx->clock_khz;
    if (name_buf && name_len) snprintf(name_buf, name_len, "%s", ctx->name);
    return DL4S_HIP_OK;
}

int dl4s_hip_timer_begin(dl4s_hip_ctx *ctx) {
    DL4S_CHECK_CTX(ctx);
    DL4S_NOT_WHILE_CAPTURING(ctx);
    DL4S_HIP_TRY(hipEventRecord(ctx->ev_begin, ctx->stream));
    return DL4S_HIP_OK;
}

int dl4s_hip_timer_end(dl4s_hip_ctx *ctx, float *out_ms) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(out_ms, DL4S_HIP_EINVALID_ARG, "dl4s_hip_timer_end: out_ms is NULL");
    DL4S_NOT_WHILE_CAPTURING(ctx);
    DL4S_HIP_TRY(hipEventRecord(ctx->ev_end, ctx->stream));
    DL4S_HIP_TRY(hipEventSynchronize(ctx->ev_end));
    DL4S_HIP_TRY(hipEventElapsedTime(out_ms, ctx->ev_begin, ctx->ev_end));
    return DL4S_HIP_OK;
}

static void release_held(dl4s_hip_ctx *ctx, std::vector<std::pair<void *, size_t>> &held) {
    std::lock_guard<std::mutex> lock(ctx->mu);
    for (auto &b : held) {
        ctx->pool[b.second].push_back(b.first);
        ctx->bytes_pooled += b.second;
        ctx->bytes_held -= b.second;
    }
    held.clear();
}

int dl4s_hip_graph_supported(void) {
    // rocprofv3 (ROCm 7.2) intercepts the queues of the process; a graph launch then ends in
    // HSA_STATUS_ERROR_INVALID_PACKET_FORMAT and an aborted queue.  Its launcher exports these variables.
    return !(getenv("ROCP_TOOL_LIBRARIES") || getenv("ROCPROFILER_LIBRARY_CTOR"));
}

int dl4s_hip_graph_begin(dl4s_hip_ctx *ctx) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(!ctx->capturing, DL4S_HIP_EINVALID_ARG, "dl4s_hip_graph_begin: a graph is being recorded already");
    DL4S_REQUIRE(dl4s_hip_graph_supported(), DL4S_HIP_EUNSUPPORTED,
                 "dl4s_hip_graph_begin: the process runs under rocprofv3, whose queue interception aborts the queue on a graph launch");
    // thread-local mode: calls of other host threads on other streams are left alone
    DL4S_HIP_TRY(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    ctx->capturing = true;
    return DL4S_HIP_OK;
}

int dl4s_hip_graph_end(dl4s_hip_ctx *ctx, dl4s_hip_graph **out_graph) {
    DL4S_CHECK_CTX(ctx);
    if (out_graph) *out_graph = nullptr;
    DL4S_REQUIRE(ctx->capturing, DL4S_HIP_EINVALID_ARG, "dl4s_hip_graph_end: no graph is being recorded");
    ctx->capturing = false;
    hipGraph_t recorded = nullptr;
    {
        const hipError_t e = hipStreamEndCapture(ctx->stream, &recorded);
        if (e != hipSuccess) {
            release_held(ctx, ctx->held_by_recording);
            return hip_error(e, "hipStreamEndCapture");
        }
    }
    if (!out_graph) {  // the caller gives the recording up
        if (recorded) (void)hipGraphDestroy(recorded);
        release_held(ctx, ctx->held_by_recording);
        return DL4S_HIP_OK;
    }
    dl4s_hip_graph *g = new (std::nothrow) dl4s_hip_graph();
    if (!g) {
        (void)hipGraphDestroy(recorded);
        release_held(ctx, ctx->held_by_recording);
        return set_error(DL4S_HIP_EOOM, "dl4s_hip_graph_end: host allocation failed");
    }
    g->graph = recorded;
    hipError_t e = hipGraphInstantiate(&g->exec, recorded, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(recorded);
        delete g;
        release_held(ctx, ctx->held_by_recording);
        return hip_error(e, "hipGraphInstantiate");
    }
    {
        std::lock_guard<std::mutex> lock(ctx->mu);
        g->held.swap(ctx->held_by_recording);
    }
    size_t nodes = 0;
    (void)hipGraphGetNodes(recorded, nullptr, &nodes);
    g->nodes = nodes;
    g->owner = ctx;
    {
        std::lock_guard<std::mutex> lock(ctx->mu);
        g->scratch_generation = ctx->scratch_generation;
    }
    *out_graph = g;
    return DL4S_HIP_OK;
}

int dl4s_hip_graph_launch(dl4s_hip_ctx *ctx, dl4s_hip_graph *graph) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(graph && graph->owner == ctx, DL4S_HIP_EINVALID_ARG,
                 "dl4s_hip_graph_launch: the graph is NULL or was recorded on another context");
    DL4S_REQUIRE(!ctx->capturing, DL4S_HIP_EINVALID_ARG, "dl4s_hip_graph_launch: a graph is being recorded");
    // the mutex orders the replay against a host thread whose call regrows the scratch block
    std::lock_guard<std::mutex> scratch_lock(ctx->scratch_mu);
    {
        std::lock_guard<std::mutex> lock(ctx->mu);
        DL4S_REQUIRE(graph->scratch_generation == ctx->scratch_generation, DL4S_HIP_EUNSUPPORTED,
                     "dl4s_hip_graph_launch: the library's scratch block has been regrown since the graph was recorded; "
                     "record it again");
    }
    DL4S_HIP_TRY(hipGraphLaunch(graph->exec, ctx->stream));
    return DL4S_HIP_OK;
}

int dl4s_hip_graph_node_count(dl4s_hip_ctx *ctx, const dl4s_hip_graph *graph, size_t *out_nodes) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(graph && out_nodes, DL4S_HIP_EINVALID_ARG, "dl4s_hip_graph_node_count: NULL argument");
    *out_nodes = graph->nodes;
    return DL4S_HIP_OK;
}

int dl4s_hip_graph_destroy(dl4s_hip_ctx *ctx, dl4s_hip_graph *graph) {
    DL4S_CHECK_CTX(ctx);
    if (!graph) return DL4S_HIP_OK;
    DL4S_REQUIRE(graph->owner == ctx, DL4S_HIP_EINVALID_ARG, "dl4s_hip_graph_destroy: recorded on another context");
    // a replay that is still running reads the executable graph
    DL4S_HIP_TRY(hipStreamSynchronize(ctx->stream));
    (void)hipGraphExecDestroy(graph->exec);
    (void)hipGraphDestroy(graph->graph);
    release_held(ctx, graph->held);
    delete graph;
    return DL4S_HIP_OK;
}

int dl4s_hip_alloc(dl4s_hip_ctx *ctx, size_t bytes, void **out_ptr) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(out_ptr, DL4S_HIP_EINVALID_ARG, "dl4s_hip_alloc: out_ptr is NULL");
    *out_ptr = nullptr;
    size_t sz = round_size(bytes);
    std::lock_guard<std::mutex> g(ctx->mu);
    void *p = nullptr;
    auto it = ctx->pool.find(sz);
    // While recording, a block freed earlier in the same recording is taken first: inside one graph the recorded calls run
    // in order, so such reuse is as safe as it is between calls issued one by one.
    auto held = ctx->held_by_recording.end();
    if (ctx->capturing)
        for (auto h = ctx->held_by_recording.begin(); h != ctx->held_by_recording.end(); ++h)
            if (h->second == sz) { held = h; break; }
    if (held != ctx->held_by_recording.end()) {
        p = held->first;
        ctx->bytes_held -= sz;
        *held = ctx->held_by_recording.back();
        ctx->held_by_recording.pop_back();
    } else if (it != ctx->pool.end() && !it->second.empty()) {
        p = it->second.back();
        it->second.pop_back();
        ctx->bytes_pooled -= sz;
    } else {
        DL4S_REQUIRE(!ctx->capturing, DL4S_HIP_EUNSUPPORTED,
                     "dl4s_hip_alloc: no pooled block of %zu bytes while a graph is being recorded; allocate before "
                     "dl4s_hip_graph_begin", sz);
        hipError_t e = hipMalloc(&p, sz);
        if (e == hipErrorOutOfMemory) {
            // give the pooled blocks back to the driver and try once more
            (void)hipGetLastError();
            (void)hipStreamSynchronize(ctx->stream);
            for (auto &kv : ctx->pool) {
                for (void *q : kv.second) (void)hipFree(q);
                kv.second.clear();
            }
            ctx->bytes_pooled = 0;
            e = hipMalloc(&p, sz);
        }
        if (e != hipSuccess) return hip_error(e, "dl4s_hip_alloc(hipMalloc)");
    }
    ctx->live[reinterpret_cast<uintptr_t>(p)] = sz;
    ctx->bytes_in_use += sz;
    *out_ptr = p;
    return DL4S_HIP_OK;
}

int dl4s_hip_free(dl4s_hip_ctx *ctx, void *ptr) {
    DL4S_CHECK_CTX(ctx);
    if (!ptr) return DL4S_HIP_OK;
    std::lock_guard<std::mutex> g(ctx->mu);
    auto it = ctx->live.find(reinterpret_cast<uintptr_t>(ptr));
    DL4S_REQUIRE(it != ctx->live.end(), DL4S_HIP_EINVALID_ARG,
                 "dl4s_hip_free: %p is not the base of a live allocation (double free or offset view)", ptr);
    size_t sz = it->second;
    ctx->live.erase(it);
    ctx->bytes_in_use -= sz;
    if (ctx->capturing) {   // the recorded kernels use the block on every replay: not reusable before the graph is gone
        ctx->held_by_recording.emplace_back(ptr, sz);
        ctx->bytes_held += sz;
        return DL4S_HIP_OK;
    }
    ctx->pool[sz].push_back(ptr);
    ctx->bytes_pooled += sz;
    return DL4S_HIP_OK;
}

int dl4s_hip_get_size(dl4s_hip_ctx *ctx, const void *ptr, size_t *out_bytes) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(ptr && out_bytes, DL4S_HIP_EINVALID_ARG, "dl4s_hip_get_size: NULL argument");
    std::lock_guard<std::mutex> g(ctx->mu);
    uintptr_t a = reinterpret_cast<uintptr_t>(ptr);
    auto it = ctx->live.upper_bound(a);
    DL4S_REQUIRE(it != ctx->live.begin(), DL4S_HIP_EINVALID_ARG, "dl4s_hip_get_size: %p is not inside a live allocation", ptr);
    --it;
    DL4S_REQUIRE(a < it->first + it->second, DL4S_HIP_EINVALID_ARG, "dl4s_hip_get_size: %p is not inside a live allocation", ptr);
    *out_bytes = it->first + it->second - a;
    return DL4S_HIP_OK;
}

int dl4s_hip_pool_trim(dl4s_hip_ctx *ctx, size_t keep_bytes) {
    DL4S_CHECK_CTX(ctx);
    DL4S_NOT_WHILE_CAPTURING(ctx);
    DL4S_HIP_TRY(hipStreamSynchronize(ctx->stream));
    std::lock_guard<std::mutex> g(ctx->mu);
    // the pool is keyed by block size: walk the sizes from the largest down
    std::vector<size_t> sizes;
    for (const auto &kv : ctx->pool)
        if (!kv.second.empty()) sizes.push_back(kv.first);
    std::sort(sizes.begin(), sizes.end(), std::greater<size_t>());
    for (size_t sz : sizes) {
        std::vector<void *> &blocks = ctx->pool[sz];
        while (!blocks.empty() && ctx->bytes_pooled > keep_bytes) {
            DL4S_HIP_TRY(hipFree(blocks.back()));
            blocks.pop_back();
            ctx->bytes_pooled -= sz;
        }
    }
    return DL4S_HIP_OK;
}

int dl4s_hip_mem_stats(dl4s_hip_ctx *ctx, size_t *out_bytes_in_use, size_t *out_bytes_pooled) {
    DL4S_CHECK_CTX(ctx);
    std::lock_guard<std::mutex> g(ctx->mu);
    if (out_bytes_in_use) *out_bytes_in_use = ctx->bytes_in_use;
    if (out_bytes_pooled) *out_bytes_pooled = ctx->bytes_pooled;
    return DL4S_HIP_OK;
}

int dl4s_hip_assign_h2d(dl4s_hip_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes) {
    DL4S_CHECK_CTX(ctx);
    if (bytes == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(dst_dev && src_host, DL4S_HIP_EINVALID_ARG, "dl4s_hip_assign_h2d: NULL pointer");
    DL4S_NOT_WHILE_CAPTURING(ctx);
    // pageable source: the async copy stages the data before returning only for small sizes, so wait
    DL4S_HIP_TRY(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
    DL4S_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return DL4S_HIP_OK;
}

int dl4s_hip_assign_d2d(dl4s_hip_ctx *ctx, void *dst_dev, const void *src_dev, size_t bytes) {
    DL4S_CHECK_CTX(ctx);
    if (bytes == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(dst_dev && src_dev, DL4S_HIP_EINVALID_ARG, "dl4s_hip_assign_d2d: NULL pointer");
    DL4S_HIP_TRY(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return DL4S_HIP_OK;
}

int dl4s_hip_assign_d2h(dl4s_hip_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes) {
    DL4S_CHECK_CTX(ctx);
    if (bytes == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(dst_host && src_dev, DL4S_HIP_EINVALID_ARG, "dl4s_hip_assign_d2h: NULL pointer");
    DL4S_NOT_WHILE_CAPTURING(ctx);
    DL4S_HIP_TRY(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    DL4S_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return DL4S_HIP_OK;
}

int dl4s_hip_get_value_f32(dl4s_hip_ctx *ctx, const float *src_dev, float *out_value) {
    return dl4s_hip_assign_d2h(ctx, out_value, src_dev, sizeof(float));
}

int dl4s_hip_set_pointee_f32(dl4s_hip_ctx *ctx, float *dst_dev, float value) {
    return dl4s_hip_assign_h2d(ctx, dst_dev, &value, sizeof(float));
}

}  // extern "C"
