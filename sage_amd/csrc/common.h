// Shared host-side declarations of the gfx950 backend: context, error plumbing, tensor helpers.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <map>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/sage_hip.h"

struct sg_block {
    uint64_t size;       // bytes held from the device for this block
    uint64_t requested;  // bytes the caller asked for (what the capacity check counts)
};

struct sg_jit_kernel {
    hipModule_t module;
    hipFunction_t fn;
};

// What a repeat call of the same map operator needs: the built kernel and the dtype its expression yields.
struct sg_map_entry {
    hipFunction_t fn;
    int result_dtype;
};

// The chunked allocator behind sg_ctx_create_pooled (Pool, memory.rs:199-475): free blocks of the two size classes,
// each a range of one device allocation ("chunk"); blocks handed out are kept by address.
struct sg_pool_block {
    char *base;       // the chunk
    uint64_t cap;     // bytes of the chunk
    uint64_t size;    // bytes of this block
    uint64_t offset;  // where it starts inside the chunk
    uint64_t age;     // requests to its pool it has sat through (Counter, memory.rs:754-786)
    bool whole() const { return size == cap; }  // !Block::is_split (memory.rs:749-751)
};
struct sg_pool {
    bool sub_buffers = true;
    std::vector<sg_pool_block> small, large;  // free blocks, in the order they were put back
    std::unordered_map<void *, sg_pool_block> live;
    uint64_t total = 0, used = 0, peak = 0;   // mem_total, mem_used, mem_peak (memory.rs:217-219)
};

// Context (session/context.rs:25-36): device + stream + kernel cache + allocator.
struct sg_ctx {
    sg_pool *pool = nullptr;  // set by sg_ctx_create_pooled with use_cache: sg_alloc / sg_free / sg_trim go through it
    int device = 0;
    hipStream_t stream = nullptr;
    int num_cus = 256;
    // allocator: live blocks by pointer, cached free blocks by size
    uint64_t capacity = 0;  // 0 = unbounded
    uint64_t used = 0;      // bytes handed out
    uint64_t reserved = 0;  // bytes held from the device (used + cached)
    uint64_t peak = 0;
    std::unordered_map<void *, sg_block> live;
    std::multimap<uint64_t, void *> cache;
    // run-time built kernels keyed by their full source text (session/context.rs:62-83)
    std::unordered_map<std::string, sg_jit_kernel> jit;
    // the same kernels by operator signature (expression program, operand dtypes and layout classes): a repeat
    // call of an operator finds its kernel without generating the source text again (CachedAccess::load_program,
    // session/context.rs:158-180); entries point into `jit`, which owns the modules
    std::unordered_map<std::string, sg_map_entry> map_by_signature;
    // stream capture (sg_graph_begin .. sg_graph_end): blocks allocated AND freed inside the captured
    // region are workspaces whose addresses are baked into the graph; they stay live with the graph
    bool capturing = false;
    // Measurement switches, read from the environment ONCE, when the context is created (so that two replays of
    // one recorded program cannot round differently because the environment changed in between):
    // SAGE_GEMM_SPLITK (1..128 k ranges, 0 = the heuristic), SAGE_GEMM_TILE (0..3, -1 = the heuristic),
    // SAGE_ATTENTION_SPLIT (0/1, -1 = the heuristic), SAGE_GEMM_DIRECT (0 = staged epilogue only).
    int force_gemm_split = 0, force_gemm_tile = -1, force_attention_split = -1;
    int gemm_direct = 1;  // SAGE_GEMM_DIRECT=0: products always leave through the staged epilogue
    int last_gemm[8] = {0, 0, 0, 0, 0, 0, 0, 0};  // template arguments of the most recent product kernel (BM 0: none yet)
    std::vector<void *> capture_allocs, capture_held;
    // errors
    std::string last_error;
    uint64_t oom_needed = 0, oom_total = 0;
};

struct sg_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    std::vector<void *> held;  // workspaces the captured kernels use on every replay
};

int sg_fail(sg_ctx *ctx, int code, const char *fmt, ...);

#define SG_HIP(ctx, expr)                                                                          \
    do {                                                                                           \
        hipError_t e_ = (expr);                                                                    \
        if (e_ != hipSuccess)                                                                      \
            return sg_fail(ctx, SG_ERR_DEVICE, "%s failed: %s (%s:%d)", #expr,                    \
                           hipGetErrorString(e_), __FILE__, __LINE__);                             \
    } while (0)

#define SG_CHECK_LAUNCH(ctx, what)                                                                 \
    do {                                                                                           \
        hipError_t e_ = hipGetLastError();                                                         \
        if (e_ != hipSuccess)                                                                      \
            return sg_fail(ctx, SG_ERR_DEVICE, "launch of %s failed: %s", what,                   \
                           hipGetErrorString(e_));                                                 \
    } while (0)

static inline int64_t sg_numel(const sg_tensor *t) {
    int64_t n = 1;
    for (int i = 0; i < t->rank; ++i) n *= t->extents[i];
    return n;
}

static inline bool sg_dtype_ok(int dt) { return dt == SG_FLOAT || dt == SG_INT || dt == SG_UINT; }

// Shape::default_strides (shape.rs:45-54)
static inline void sg_default_strides(const int64_t *ext, int rank, int64_t *out) {
    int64_t size = 1;
    for (int i = 0; i < rank; ++i) size *= ext[i];
    for (int i = 0; i < rank; ++i) {
        size /= ext[i] ? ext[i] : 1;
        out[i] = size;
    }
}

// Dense row-major at any offset.  Axes of extent 1 may carry any stride.
static inline bool sg_is_dense(const sg_tensor *t) {
    int64_t expect = 1;
    for (int i = t->rank - 1; i >= 0; --i) {
        if (t->extents[i] != 1 && t->strides[i] != expect) return false;
        expect *= t->extents[i];
    }
    return true;
}

int sg_validate_tensor(sg_ctx *ctx, const sg_tensor *t, const char *name);

// pool.cpp: the chunked allocator (sg_ctx::pool)
int sg_pool_alloc(sg_ctx *ctx, uint64_t nbytes, void **dptr);
int sg_pool_free(sg_ctx *ctx, void *dptr);
int sg_pool_trim(sg_ctx *ctx);
void sg_pool_destroy(sg_ctx *ctx);

// gemm.hip: per-device set-up (the address of the static split-K scratch), run by sg_ctx_create.
int sg_gemm_device_setup(sg_ctx *ctx);

// A kernel that moves at least 16 MiB streams them: a consumer's workgroups sit on any of the 8 XCDs, so what a
// kernel leaves in one XCD's L2 serves an eighth of its readers at best, while stores that stay dirty in the L2s are
// written back in one burst when the kernel ends; non-temporal loads and stores (no allocation in the L2s on the
// way through) sustain about a fifth more HBM bandwidth.  SAGE_STREAM_MIN_BYTES overrides the threshold
// (0 = always stream); BERT-base b32 x s128, whose LayerNorms move 25 MB each: 5.731 -> 5.717 ms per step.
bool sg_streaming(int64_t bytes);

// Magic-number unsigned division for n < 2^31: q = (umulhi(n, magic) + n) >> shift.
struct sg_fastdiv {
    uint32_t magic, shift;
};
static inline sg_fastdiv sg_make_fastdiv(uint32_t d) {
    sg_fastdiv f;
    uint32_t s = 0;
    while (s < 32 && (1ull << s) < d) ++s;
    f.shift = s;
    f.magic = (uint32_t)(((1ull << 32) * ((1ull << s) - d)) / d + 1);
    return f;
}
