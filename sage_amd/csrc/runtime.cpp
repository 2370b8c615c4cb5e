// Context, allocator and transfers of the gfx950 backend.
//
// Stands in for the reference's device seam: Device::new / alloc_buffer, Buffer::{read,write,fill}
// (session/device.rs:45-191), Context::alloc (session/context.rs:119-137) and the capacity
// accounting of Pool::alloc / check_space (session/memory.rs:246-255, 353-362).
#include "common.h"

#include <cstdlib>
#include <cstring>

int sg_fail(sg_ctx *ctx, int code, const char *fmt, ...) {
    if (ctx) {
        char buf[2048];
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(buf, sizeof buf, fmt, ap);
        va_end(ap);
        ctx->last_error = buf;
    }
    return code;
}

bool sg_streaming(int64_t bytes) {
    static const int64_t min_bytes = [] {
        const char *e = getenv("SAGE_STREAM_MIN_BYTES");
        return e ? (int64_t)strtoll(e, nullptr, 10) : (int64_t)16 << 20;
    }();
    return bytes >= min_bytes;
}

int sg_validate_tensor(sg_ctx *ctx, const sg_tensor *t, const char *name) {
    if (!t) return sg_fail(ctx, SG_ERR_ARG, "%s: null tensor", name);
    if (!t->base) return sg_fail(ctx, SG_ERR_ARG, "%s: null base pointer", name);
    if (t->rank < 1 || t->rank > SG_MAX_RANK)
        return sg_fail(ctx, SG_ERR_SHAPE, "%s: rank %d outside 1..%d", name, t->rank, SG_MAX_RANK);
    if (!sg_dtype_ok(t->dtype))
        return sg_fail(ctx, SG_ERR_DTYPE, "%s: dtype %d is not a 4-byte type this backend computes on", name, t->dtype);
    int64_t n = 1;
    for (int i = 0; i < t->rank; ++i) {
        if (t->extents[i] < 1) return sg_fail(ctx, SG_ERR_SHAPE, "%s: extent[%d] = %lld", name, i, (long long)t->extents[i]);
        if (t->strides[i] < 0) return sg_fail(ctx, SG_ERR_SHAPE, "%s: negative stride", name);
        n *= t->extents[i];
        if (n >= (1ll << 31)) return sg_fail(ctx, SG_ERR_SHAPE, "%s: more than 2^31-1 elements", name);
    }
    if (t->offset < 0) return sg_fail(ctx, SG_ERR_SHAPE, "%s: negative offset", name);
    // the generated index arithmetic is 32-bit unsigned, as the reference's is (core.rs:133-168)
    int64_t last = t->offset;
    for (int i = 0; i < t->rank; ++i) last += (t->extents[i] - 1) * t->strides[i];
    if (last >= (1ll << 32)) return sg_fail(ctx, SG_ERR_SHAPE, "%s: addresses beyond 2^32 elements", name);
    return SG_OK;
}

extern "C" {

int sg_ctx_create(int device_idx, uint64_t capacity_bytes, sg_ctx **out) {
    if (!out) return SG_ERR_ARG;
    *out = nullptr;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) return SG_ERR_DEVICE;
    if (device_idx < 0 || device_idx >= count) return SG_ERR_ARG;
    if (hipSetDevice(device_idx) != hipSuccess) return SG_ERR_DEVICE;
    sg_ctx *ctx = new sg_ctx();
    ctx->device = device_idx;
    ctx->capacity = capacity_bytes;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device_idx) == hipSuccess) ctx->num_cus = prop.multiProcessorCount;
    // one in-order queue per context (session/device.rs:64), default priority
    if (hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking) != hipSuccess) {
        delete ctx;
        return SG_ERR_DEVICE;
    }
    if (const char *e = getenv("SAGE_GEMM_SPLITK")) {
        const int v = atoi(e);
        ctx->force_gemm_split = v < 1 ? 1 : v > 128 ? 128 : v;  // the second pass sums at most 128 ranges
    }
    if (const char *e = getenv("SAGE_GEMM_TILE"))
        if (e[0] >= '0' && e[0] <= '3' && e[1] == 0) ctx->force_gemm_tile = e[0] - '0';
    if (const char *e = getenv("SAGE_ATTENTION_SPLIT")) ctx->force_attention_split = atoi(e) != 0;
    if (const char *e = getenv("SAGE_GEMM_DIRECT")) ctx->gemm_direct = atoi(e) != 0;
    if (sg_gemm_device_setup(ctx) != SG_OK) {
        (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return SG_ERR_DEVICE;
    }
    *out = ctx;
    return SG_OK;
}

int sg_ctx_create_pooled(int device_idx, uint64_t capacity_bytes, int use_cache, int use_sub_buffer, sg_ctx **out) {
    const int rc = sg_ctx_create(device_idx, capacity_bytes, out);
    if (rc != SG_OK || !use_cache) return rc;
    (*out)->pool = new sg_pool();
    (*out)->pool->sub_buffers = use_sub_buffer != 0;
    return SG_OK;
}

int sg_trim(sg_ctx *ctx) {
    if (!ctx) return SG_ERR_ARG;
    if (ctx->pool) return sg_pool_trim(ctx);
    if (ctx->cache.empty()) return SG_OK;
    if (ctx->capturing) return sg_fail(ctx, SG_ERR_ARG, "sg_trim waits for the stream and cannot be captured into a graph");
    SG_HIP(ctx, hipStreamSynchronize(ctx->stream));
    for (auto &kv : ctx->cache) {
        (void)hipFree(kv.second);
        ctx->reserved -= kv.first;
    }
    ctx->cache.clear();
    return SG_OK;
}

int sg_ctx_destroy(sg_ctx *ctx) {
    if (!ctx) return SG_ERR_ARG;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    for (auto &kv : ctx->jit) (void)hipModuleUnload(kv.second.module);
    for (auto &kv : ctx->cache) (void)hipFree(kv.second);
    for (auto &kv : ctx->live) (void)hipFree(kv.first);
    sg_pool_destroy(ctx);
    (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return SG_OK;
}

static uint64_t round_block(uint64_t n) {
    if (n == 0) n = 1;
    const uint64_t small_round = 512, large_round = 2ull << 20;
    if (n < (1ull << 20)) return (n + small_round - 1) / small_round * small_round;
    return (n + large_round - 1) / large_round * large_round;
}

int sg_alloc(sg_ctx *ctx, uint64_t nbytes, void **dptr) {
    if (!ctx || !dptr) return SG_ERR_ARG;
    *dptr = nullptr;
    if (ctx->pool) return sg_pool_alloc(ctx, nbytes, dptr);
    // Pool::check_space (memory.rs:246-255)
    if (ctx->capacity && ctx->used + nbytes > ctx->capacity) {
        ctx->oom_needed = ctx->used + nbytes - ctx->capacity;
        ctx->oom_total = ctx->used;
        return sg_fail(ctx, SG_ERR_OOM, "tried to allocate %llu bytes: %llu more than the capacity allows, %llu in use",
                       (unsigned long long)nbytes, (unsigned long long)ctx->oom_needed, (unsigned long long)ctx->oom_total);
    }
    uint64_t sz = round_block(nbytes);
    void *p = nullptr;
    auto it = ctx->cache.lower_bound(sz);
    if (it != ctx->cache.end() && it->first <= sz + sz / 4) {
        p = it->second;
        sz = it->first;
        ctx->cache.erase(it);
    } else {
        hipError_t e = hipMalloc(&p, sz);
        if (e != hipSuccess && !ctx->capturing) {  // trimming synchronises, which a capture forbids
            (void)hipGetLastError();
            int rc = sg_trim(ctx);
            if (rc != SG_OK) return rc;
            e = hipMalloc(&p, sz);
        }
        if (e != hipSuccess) {
            (void)hipGetLastError();
            ctx->oom_needed = nbytes;
            ctx->oom_total = ctx->used;
            return sg_fail(ctx, SG_ERR_OOM, "device refused %llu bytes (%s), %llu in use",
                           (unsigned long long)sz, hipGetErrorString(e), (unsigned long long)ctx->used);
        }
        ctx->reserved += sz;
    }
    ctx->live[p] = sg_block{sz, nbytes};
    if (ctx->capturing) ctx->capture_allocs.push_back(p);
    ctx->used += nbytes;
    if (ctx->used > ctx->peak) ctx->peak = ctx->used;
    *dptr = p;
    return SG_OK;
}

int sg_free(sg_ctx *ctx, void *dptr) {
    if (!ctx) return SG_ERR_ARG;
    if (!dptr) return SG_OK;
    if (ctx->pool) return sg_pool_free(ctx, dptr);
    auto it = ctx->live.find(dptr);
    if (it == ctx->live.end()) return sg_fail(ctx, SG_ERR_ARG, "sg_free: %p was not allocated by this context", dptr);
    if (ctx->capturing) {
        for (void *q : ctx->capture_allocs)
            if (q == dptr) {  // a workspace of the captured kernels: it belongs to the graph from now on
                ctx->capture_held.push_back(dptr);
                return SG_OK;
            }
    }
    ctx->used -= it->second.requested;
    // Work already queued on the context's in-order stream finishes before any later launch that
    // is handed this block again, so the block can be reused without a device synchronisation.
    ctx->cache.emplace(it->second.size, dptr);
    ctx->live.erase(it);
    return SG_OK;
}

int sg_mem_stats(sg_ctx *ctx, uint64_t *used, uint64_t *reserved, uint64_t *peak, uint64_t *capacity) {
    if (!ctx) return SG_ERR_ARG;
    if (ctx->pool) {
        if (used) *used = ctx->pool->used;
        if (reserved) *reserved = ctx->pool->total;
        if (peak) *peak = ctx->pool->peak;
        if (capacity) *capacity = ctx->capacity;
        return SG_OK;
    }
    if (used) *used = ctx->used;
    if (reserved) *reserved = ctx->reserved;
    if (peak) *peak = ctx->peak;
    if (capacity) *capacity = ctx->capacity;
    return SG_OK;
}

int sg_memcpy_h2d(sg_ctx *ctx, void *dst_dev, const void *src_host, uint64_t nbytes) {
    if (!ctx || (!dst_dev && nbytes) || (!src_host && nbytes)) return SG_ERR_ARG;
    if (!nbytes) return SG_OK;
    if (ctx->capturing) return sg_fail(ctx, SG_ERR_ARG, "sg_memcpy_h2d waits for the stream and cannot be captured into a graph");
    SG_HIP(ctx, hipMemcpyAsync(dst_dev, src_host, nbytes, hipMemcpyHostToDevice, ctx->stream));
    SG_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return SG_OK;
}

int sg_memcpy_d2h(sg_ctx *ctx, void *dst_host, const void *src_dev, uint64_t nbytes) {
    if (!ctx || (!dst_host && nbytes) || (!src_dev && nbytes)) return SG_ERR_ARG;
    if (!nbytes) return SG_OK;
    if (ctx->capturing) return sg_fail(ctx, SG_ERR_ARG, "sg_memcpy_d2h waits for the stream and cannot be captured into a graph");
    SG_HIP(ctx, hipMemcpyAsync(dst_host, src_dev, nbytes, hipMemcpyDeviceToHost, ctx->stream));
    SG_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return SG_OK;
}

int sg_memcpy_d2d(sg_ctx *ctx, void *dst_dev, const void *src_dev, uint64_t nbytes) {
    if (!ctx || (!dst_dev && nbytes) || (!src_dev && nbytes)) return SG_ERR_ARG;
    if (!nbytes) return SG_OK;
    SG_HIP(ctx, hipMemcpyAsync(dst_dev, src_dev, nbytes, hipMemcpyDeviceToDevice, ctx->stream));
    return SG_OK;
}

int sg_sync(sg_ctx *ctx) {
    if (!ctx) return SG_ERR_ARG;
    if (ctx->capturing) return sg_fail(ctx, SG_ERR_ARG, "sg_sync waits for the stream and cannot be captured into a graph");
    SG_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return SG_OK;
}

void *sg_stream(sg_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

int sg_event_create(sg_ctx *ctx, void **event) {
    if (!ctx || !event) return SG_ERR_ARG;
    hipEvent_t e;
    SG_HIP(ctx, hipEventCreate(&e));
    *event = (void *)e;
    return SG_OK;
}

int sg_event_record(sg_ctx *ctx, void *event) {
    if (!ctx || !event) return SG_ERR_ARG;
    SG_HIP(ctx, hipEventRecord((hipEvent_t)event, ctx->stream));
    return SG_OK;
}

int sg_event_elapsed_ms(sg_ctx *ctx, void *start, void *stop, float *ms) {
    if (!ctx || !start || !stop || !ms) return SG_ERR_ARG;
    SG_HIP(ctx, hipEventSynchronize((hipEvent_t)stop));
    SG_HIP(ctx, hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return SG_OK;
}

int sg_event_destroy(sg_ctx *ctx, void *event) {
    if (!ctx || !event) return SG_ERR_ARG;
    SG_HIP(ctx, hipEventDestroy((hipEvent_t)event));
    return SG_OK;
}

const char *sg_last_error(sg_ctx *ctx) { return ctx ? ctx->last_error.c_str() : "null context"; }

int sg_last_oom(sg_ctx *ctx, uint64_t *needed, uint64_t *total) {
    if (!ctx) return SG_ERR_ARG;
    if (needed) *needed = ctx->oom_needed;
    if (total) *total = ctx->oom_total;
    return SG_OK;
}

int sg_kernel_cache_size(sg_ctx *ctx) { return ctx ? (int)ctx->jit.size() : -1; }

}  // extern "C"

// ---- HIP graphs: a recorded sequence of launches replayed with one submission ---------------------
// The reference replays a compiled Program launch by launch (session.rs:208-468); a launch-bound
// program (dozens of microsecond kernels) is bounded by that host loop.  Everything the library
// launches goes to the context's stream, so a stream capture between begin and end records it.

int sg_graph_begin(sg_ctx *ctx) {
    if (!ctx) return SG_ERR_ARG;
    if (ctx->capturing) return sg_fail(ctx, SG_ERR_ARG, "sg_graph_begin: a capture is already open");
    SG_HIP(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed));
    ctx->capturing = true;
    ctx->capture_allocs.clear();
    ctx->capture_held.clear();
    return SG_OK;
}

int sg_graph_end(sg_ctx *ctx, sg_graph **out) {
    if (!ctx || !out) return SG_ERR_ARG;
    *out = nullptr;
    if (!ctx->capturing) return sg_fail(ctx, SG_ERR_ARG, "sg_graph_end: no capture is open");
    ctx->capturing = false;
    sg_graph *g = new sg_graph();
    g->held.swap(ctx->capture_held);
    ctx->capture_allocs.clear();
    hipError_t e = hipStreamEndCapture(ctx->stream, &g->graph);
    if (e == hipSuccess) e = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        if (g->graph) (void)hipGraphDestroy(g->graph);
        for (void *p : g->held) (void)sg_free(ctx, p);
        delete g;
        return sg_fail(ctx, SG_ERR_DEVICE, "graph capture failed: %s", hipGetErrorString(e));
    }
    *out = g;
    return SG_OK;
}

int sg_graph_launch(sg_ctx *ctx, sg_graph *g) {
    if (!ctx || !g || !g->exec) return SG_ERR_ARG;
    if (ctx->capturing) return sg_fail(ctx, SG_ERR_ARG, "sg_graph_launch inside a capture");
    SG_HIP(ctx, hipGraphLaunch(g->exec, ctx->stream));
    return SG_OK;
}

int sg_graph_destroy(sg_ctx *ctx, sg_graph *g) {
    if (!ctx) return SG_ERR_ARG;
    if (!g) return SG_OK;
    (void)hipStreamSynchronize(ctx->stream);  // a replay may still be running on the held workspaces
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    for (void *p : g->held) (void)sg_free(ctx, p);
    delete g;
    return SG_OK;
}
