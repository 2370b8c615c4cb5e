// The chunked, caching device allocator: the caching branch of the reference's Pool (session/memory.rs:199-475),
// which its Context leaves switched off (context.rs:49) and sg_ctx_create_pooled switches on.
//
// What is kept of the reference: the two size classes and their chunk sizes, the choice of the smallest free
// block that fits and is not wastefully large, the split thresholds, ages counted in requests, collection of
// whole free chunks above the average age once 80 % of the capacity is in use, and the release of the largest
// whole free chunks when the capacity forbids a new one.  A block is a (chunk, offset, size) triple and the
// address handed out is chunk + offset: device memory is one flat address space here, there is no sub-buffer
// object to create.
// Where the reference's text cannot be meant as written, this file does what the surrounding code intends:
//   * merging a freed block with its free neighbours adds their sizes (memory.rs:381-385 keeps the largest of
//     them, which loses the rest of the chunk for good);
//   * a freed block returns to the class its chunk was taken for (memory.rs:367 picks the class by the chunk's
//     size, which is never below the small-class limit, so every block would end up in the large class);
//   * collection and release give their bytes back to the total the capacity bounds (memory.rs:403-475 never
//     subtract them);
//   * without sub-buffers a free chunk can still be handed out whole (the filter at memory.rs:303-308 rejects
//     every block then).
#include "common.h"

#include <algorithm>

namespace {

constexpr uint64_t KIB = 1024, MIB = 1024 * 1024;
constexpr uint64_t ALIGN = 256;               // every block starts where a device allocation could
constexpr uint64_t MIN_BLOCK = 512;           // MIN_BLOCK_SIZE   (memory.rs:23, there in 4-byte elements)
constexpr uint64_t SMALL_SIZE = 1 * MIB;      // SMALL_SIZE       (memory.rs:25)
constexpr uint64_t SMALL_BUFFER = 2 * MIB;    // SMALL_BUFFER     (memory.rs:27)
constexpr uint64_t LARGE_BUFFER = 20 * MIB;   // LARGE_BUFFER     (memory.rs:29)
constexpr uint64_t MIN_LARGE = 10 * MIB;      // MIN_LARGE_ALLOC  (memory.rs:31)
constexpr uint64_t ROUND_LARGE = 2 * MIB;     // ROUND_LARGE      (memory.rs:33)
constexpr uint64_t SPLIT_LIM = 2 * LARGE_BUFFER;  // SPLIT_LIM    (memory.rs:35)

std::vector<sg_pool_block> &class_of_request(sg_pool &p, uint64_t size) { return size < SMALL_SIZE ? p.small : p.large; }  // select_pool
std::vector<sg_pool_block> &class_of_chunk(sg_pool &p, uint64_t cap) { return cap == SMALL_BUFFER ? p.small : p.large; }

// Pool::allocation_size (memory.rs:257-265)
uint64_t chunk_size(uint64_t size) {
    if (size < SMALL_SIZE) return SMALL_BUFFER;
    if (size < MIN_LARGE) return LARGE_BUFFER;
    return (size + ROUND_LARGE - 1) / ROUND_LARGE * ROUND_LARGE;
}

// Pool::check_space (memory.rs:246-255) on the bytes held from the device
bool over_capacity(sg_ctx *ctx, uint64_t more) {
    sg_pool &p = *ctx->pool;
    if (!ctx->capacity || p.total + more <= ctx->capacity) return false;
    ctx->oom_needed = p.total + more - ctx->capacity;
    ctx->oom_total = p.total;
    return true;
}

// Pool::expand (memory.rs:267-283): one more chunk for the class of this request
int expand(sg_ctx *ctx, uint64_t size) {
    sg_pool &p = *ctx->pool;
    const uint64_t bytes = chunk_size(size);
    if (over_capacity(ctx, bytes)) return SG_ERR_OOM;
    void *base = nullptr;
    const hipError_t e = hipMalloc(&base, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        ctx->oom_needed = bytes;
        ctx->oom_total = p.total;
        return SG_ERR_OOM;
    }
    class_of_request(p, size).push_back(sg_pool_block{(char *)base, bytes, bytes, 0, 0});
    p.total += bytes;
    if (p.total > p.peak) p.peak = p.total;
    return SG_OK;
}

// Pool::get_free_block (memory.rs:285-331)
bool take_free_block(sg_pool &p, uint64_t size, sg_pool_block *out) {
    std::vector<sg_pool_block> &cls = class_of_request(p, size);
    for (sg_pool_block &b : cls) ++b.age;
    int best = -1;
    for (int i = 0; i < (int)cls.size(); ++i) {
        const sg_pool_block &b = cls[i];
        if (size > b.size) continue;
        if (!p.sub_buffers && !b.whole()) continue;
        // not a huge block for a modest request, nor one far beyond a huge request (memory.rs:305-307)
        if ((size < SPLIT_LIM && SPLIT_LIM <= b.size) || (SPLIT_LIM <= size && size + LARGE_BUFFER <= b.size)) continue;
        if (best < 0 || b.size < cls[best].size) best = i;  // the first of the smallest (Iterator::min_by_key)
    }
    if (best < 0) return false;
    sg_pool_block b = cls[best];
    cls.erase(cls.begin() + best);
    b.age = 0;
    const uint64_t rest = b.size - size;
    const bool split = (size <= SMALL_SIZE && MIN_BLOCK <= rest) || (SMALL_SIZE < size && size < SPLIT_LIM && SMALL_SIZE < rest);
    if (split && p.sub_buffers) {  // Block::split (memory.rs:726-747): the request in front, the rest back to the class
        cls.push_back(sg_pool_block{b.base, b.cap, rest, b.offset + size, 0});
        b.size = size;
    }
    p.used += b.size;
    *out = b;
    return true;
}

// Returning chunks to the device waits for the context's stream first: whatever queued work still reads a block
// that was freed a moment ago has finished by the time its memory goes.
uint64_t drop_chunks(sg_ctx *ctx, std::vector<sg_pool_block> &cls, const std::vector<int> &idx) {
    sg_pool &p = *ctx->pool;
    uint64_t bytes = 0;
    if (!idx.empty()) (void)hipStreamSynchronize(ctx->stream);
    for (int k = (int)idx.size() - 1; k >= 0; --k) {  // indices ascending: erase from the back
        const sg_pool_block b = cls[idx[k]];
        (void)hipFree(b.base);
        bytes += b.size;
        cls.erase(cls.begin() + idx[k]);
    }
    p.total -= bytes;
    return bytes;
}

// Pool::garbage_collect (memory.rs:403-449): once 80 % of the capacity is handed out, whole free chunks of the
// large class at or above the average age go back to the device, round after round, until a fifth of the
// capacity has been reclaimed or a round frees nothing.
uint64_t collect(sg_ctx *ctx) {
    sg_pool &p = *ctx->pool;
    if (!ctx->capacity) return 0;
    const uint64_t threshold = (uint64_t)((float)ctx->capacity * 0.8f);  // GC_THRESHOLD (memory.rs:37), the reference's f32 product
    if (p.used < threshold) return 0;
    const uint64_t target = ctx->capacity - threshold;
    uint64_t total_age = 0, freeable = 0;
    for (const sg_pool_block &b : p.large)
        if (b.whole()) total_age += b.age, ++freeable;
    uint64_t reclaimed = 0;
    bool freed = true;
    while (reclaimed < target && freed && freeable > 0) {
        const uint64_t age_threshold = total_age / freeable;
        std::vector<int> idx;
        for (int i = 0; i < (int)p.large.size(); ++i)
            if (p.large[i].whole() && p.large[i].age >= age_threshold) idx.push_back(i);
        for (int i : idx) total_age -= p.large[i].age;
        freeable -= idx.size();
        freed = !idx.empty();
        reclaimed += drop_chunks(ctx, p.large, idx);
    }
    return reclaimed;
}

// Pool::release_cached_blocks (memory.rs:451-475): the largest whole free chunks of the large class, until the
// request (at least 40 MiB) has been covered
uint64_t release(sg_ctx *ctx, uint64_t size) {
    sg_pool &p = *ctx->pool;
    uint64_t released = 0;
    while (released < std::max(size, SPLIT_LIM)) {
        int best = -1;
        for (int i = 0; i < (int)p.large.size(); ++i)
            if (p.large[i].whole() && (best < 0 || p.large[i].size >= p.large[best].size)) best = i;  // the last of the largest (max_by_key)
        if (best < 0) break;
        released += drop_chunks(ctx, p.large, std::vector<int>{best});
    }
    return released;
}

}  // namespace

// Pool::alloc, caching branch (memory.rs:333-352)
int sg_pool_alloc(sg_ctx *ctx, uint64_t nbytes, void **dptr) {
    sg_pool &p = *ctx->pool;
    if (nbytes > (1ull << 48)) {  // (beyond any device; also keeps the roundings below from wrapping)
        ctx->oom_needed = nbytes;
        ctx->oom_total = p.total;
        return sg_fail(ctx, SG_ERR_OOM, "tried to allocate %llu bytes", (unsigned long long)nbytes);
    }
    const uint64_t size = (std::max<uint64_t>(nbytes, 1) + ALIGN - 1) / ALIGN * ALIGN;
    sg_pool_block b;
    if (!take_free_block(p, size, &b)) {
        // giving chunks back waits for the device, which a stream capture forbids: while capturing, only a new chunk is tried
        if (!ctx->capturing) (void)collect(ctx);
        int rc = expand(ctx, size);
        if (rc != SG_OK && !ctx->capturing) {
            (void)release(ctx, size);
            rc = expand(ctx, size);
        }
        if (rc != SG_OK && !ctx->capturing) {
            // Beyond the reference, whose release looks at the large class only: whole free chunks of the small class
            // go back too before the request is refused, so that memory a caller frees in answer to SG_ERR_OOM (the
            // evaluator's eviction loop, session.rs:259-325) can serve a request of the other class.
            std::vector<int> idx;
            for (int i = 0; i < (int)p.small.size(); ++i)
                if (p.small[i].whole()) idx.push_back(i);
            if (!idx.empty()) {
                (void)drop_chunks(ctx, p.small, idx);
                rc = expand(ctx, size);
            }
        }
        if (rc != SG_OK)
            return sg_fail(ctx, SG_ERR_OOM, "tried to take a chunk of %llu bytes for a request of %llu: %llu more than the capacity allows, %llu held",
                           (unsigned long long)chunk_size(size), (unsigned long long)nbytes, (unsigned long long)ctx->oom_needed, (unsigned long long)ctx->oom_total);
        if (!take_free_block(p, size, &b)) {  // MemoryError::NoFreeBlock (memory.rs:56-57)
            ctx->oom_needed = size;
            ctx->oom_total = p.total;
            return sg_fail(ctx, SG_ERR_OOM, "no free block left in the pool for %llu bytes", (unsigned long long)nbytes);
        }
    }
    void *ptr = b.base + b.offset;
    p.live[ptr] = b;
    if (ctx->capturing) ctx->capture_allocs.push_back(ptr);
    *dptr = ptr;
    return SG_OK;
}

// Pool::free, caching branch (memory.rs:364-396)
int sg_pool_free(sg_ctx *ctx, void *dptr) {
    sg_pool &p = *ctx->pool;
    auto it = p.live.find(dptr);
    if (it == p.live.end()) return sg_fail(ctx, SG_ERR_ARG, "sg_free: %p was not allocated by this context", dptr);
    if (ctx->capturing) {
        for (void *q : ctx->capture_allocs)
            if (q == dptr) {  // a workspace of the captured kernels: it belongs to the graph from now on
                ctx->capture_held.push_back(dptr);
                return SG_OK;
            }
    }
    sg_pool_block b = it->second;
    p.live.erase(it);
    p.used -= b.size;
    std::vector<sg_pool_block> &cls = class_of_chunk(p, b.cap);
    b.age = 0;
    if (p.sub_buffers) {
        // free neighbours inside the same chunk join the block (work queued on the context's in-order stream that
        // still uses either part finishes before any later launch that is handed the merged block)
        for (int i = (int)cls.size() - 1; i >= 0; --i) {
            const sg_pool_block &n = cls[i];
            if (n.base != b.base) continue;
            if (n.offset + n.size == b.offset) {
                b.offset = n.offset;
                b.size += n.size;
                cls.erase(cls.begin() + i);
            } else if (b.offset + b.size == n.offset) {
                b.size += n.size;
                cls.erase(cls.begin() + i);
            }
        }
    }
    cls.push_back(b);
    return SG_OK;
}

// sg_trim: every whole free chunk of both classes goes back to the device
int sg_pool_trim(sg_ctx *ctx) {
    sg_pool &p = *ctx->pool;
    if (ctx->capturing) return sg_fail(ctx, SG_ERR_ARG, "sg_trim waits for the device and cannot be captured into a graph");
    for (std::vector<sg_pool_block> *cls : {&p.small, &p.large}) {
        std::vector<int> idx;
        for (int i = 0; i < (int)cls->size(); ++i)
            if ((*cls)[i].whole()) idx.push_back(i);
        (void)drop_chunks(ctx, *cls, idx);
    }
    return SG_OK;
}

void sg_pool_destroy(sg_ctx *ctx) {
    sg_pool *p = ctx->pool;
    if (!p) return;
    // every chunk is freed once: through the block (free or handed out) that starts at its first byte
    for (std::vector<sg_pool_block> *cls : {&p->small, &p->large})
        for (const sg_pool_block &b : *cls)
            if (b.offset == 0) (void)hipFree(b.base);
    for (const auto &kv : p->live)
        if (kv.second.offset == 0) (void)hipFree(kv.second.base);
    delete p;
    ctx->pool = nullptr;
}
