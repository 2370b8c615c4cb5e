// Reductions and fused row operators for gfx950.
//
// Replaces the reference's `reduce` and `reduce_arg` kernels (reduce.rs:258-325, 372-431), which
// give every output element to ONE work-item that walks its whole reduced span serially, and the
// multi-launch compositions built on them (softmax, log-sum-exp / cross-entropy, layer_norm:
// nn.rs:42-100).  Here:
//   * a reduced span that is contiguous in memory is walked by a whole 64-lane wavefront (short
//     rows) or a 256-thread workgroup (long rows) with 16-byte loads, combined with cross-lane
//     shuffles and, across wavefronts, through LDS;
//   * any other layout keeps one thread per output, which is coalesced whenever the kept innermost
//     axis is the contiguous one (pooling over [N,OH,OW,KH,KW,C], column sums);
//   * softmax, softmax-cross-entropy and layer-norm read each row once into registers and write
//     once: 2 passes over HBM in total instead of 6-10.
// fp32 sums are tree-ordered, so they differ from the reference's serial order by rounding only.
#include "common.h"

namespace {

constexpr int WAVE = 64;

enum { OP_SUM = 0, OP_PROD = 1, OP_MAX = 2, OP_MIN = 3 };

template <class T> struct Lim;
template <> struct Lim<float> {
    __device__ static float lowest() { return -__builtin_inff(); }
    __device__ static float highest() { return __builtin_inff(); }
};
template <> struct Lim<int> {
    __device__ static int lowest() { return (int)0x80000000; }
    __device__ static int highest() { return 0x7fffffff; }
};
template <> struct Lim<unsigned> {
    __device__ static unsigned lowest() { return 0u; }
    __device__ static unsigned highest() { return 0xffffffffu; }
};

template <int OP, class T> __device__ __forceinline__ T identity() {
    if (OP == OP_SUM) return (T)0;
    if (OP == OP_PROD) return (T)1;
    if (OP == OP_MAX) return Lim<T>::lowest();
    return Lim<T>::highest();
}
// max(acc,v) = acc < v ? v : acc ; min(acc,v) = v < acc ? v : acc  (OpenCL min/max, reduce.rs:266-269)
template <int OP, class T> __device__ __forceinline__ T combine(T a, T v) {
    if (OP == OP_SUM) return a + v;
    if (OP == OP_PROD) return a * v;
    if (OP == OP_MAX) return a < v ? v : a;
    return v < a ? v : a;
}

template <class T> __device__ __forceinline__ T shfl_xor(T v, int m) { return __shfl_xor(v, m, WAVE); }

template <int OP, class T> __device__ __forceinline__ T wave_reduce(T v) {
#pragma unroll
    for (int m = WAVE / 2; m >= 1; m >>= 1) v = combine<OP, T>(v, shfl_xor(v, m));
    return v;
}

// The same over the 64 lanes for fp32 with data-parallel-primitive moves instead of LDS permutes: a butterfly step
// through ds_bpermute costs an address computation and an LDS round trip (six of them in a row, twice for a
// LayerNorm row, while the row's registers wait), a DPP move is one vector instruction.  Quad permutes give
// every lane its quad's total, two row shifts leave the row's total in lanes 12..15, two row broadcasts carry it
// across the four rows into lane 63, which is read back as a scalar.  Lanes a move does not reach receive the
// operator's identity.  (A fixed tree: the same input gives the same bits.)
template <int OP> __device__ __forceinline__ float wave_reduce_dpp(float v) {
    const int id = __builtin_bit_cast(int, identity<OP, float>());
#define SG_DPP_STEP(CTRL, ROW_MASK) \
    v = combine<OP, float>(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(id, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, false)))
    SG_DPP_STEP(0xb1, 0xf);   // quad_perm:[1,0,3,2]
    SG_DPP_STEP(0x4e, 0xf);   // quad_perm:[2,3,0,1]
    SG_DPP_STEP(0x114, 0xf);  // row_shr:4
    SG_DPP_STEP(0x118, 0xf);  // row_shr:8
    SG_DPP_STEP(0x142, 0xa);  // row_bcast:15 into rows 1 and 3
    SG_DPP_STEP(0x143, 0xc);  // row_bcast:31 into rows 2 and 3
#undef SG_DPP_STEP
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
template <> __device__ __forceinline__ float wave_reduce<OP_SUM, float>(float v) { return wave_reduce_dpp<OP_SUM>(v); }
template <> __device__ __forceinline__ float wave_reduce<OP_MAX, float>(float v) { return wave_reduce_dpp<OP_MAX>(v); }
template <> __device__ __forceinline__ float wave_reduce<OP_MIN, float>(float v) { return wave_reduce_dpp<OP_MIN>(v); }
template <> __device__ __forceinline__ float wave_reduce<OP_PROD, float>(float v) { return wave_reduce_dpp<OP_PROD>(v); }

struct Dims {
    int n;
    uint32_t ext[SG_MAX_RANK];
    uint32_t stride[SG_MAX_RANK];
    uint32_t magic[SG_MAX_RANK], shift[SG_MAX_RANK];  // division by ext[a] as a multiply-high and a shift
};

// linear index over `d.ext` (row-major) -> element offset.  No hardware division: ids are below 2^31
// (checked on the host), where q = (umulhi(id, magic) + id) >> shift is exact; the outermost axis needs
// no division at all.
__device__ __forceinline__ uint32_t decompose(const Dims &d, uint32_t id) {
    uint32_t off = 0;
    for (int a = d.n - 1; a > 0; --a) {
        const uint32_t q = (__umulhi(id, d.magic[a]) + id) >> d.shift[a];
        off += (id - q * d.ext[a]) * d.stride[a];
        id = q;
    }
    return d.n > 0 ? off + id * d.stride[0] : off;
}

// ---- one thread per output, nested walk over the reduced axes -------------------------------
template <int OP, class T>
__global__ void __launch_bounds__(256) reduce_thread_kernel(const T *__restrict__ x, T *__restrict__ y, uint32_t n_out,
                                                            uint32_t x_off, Dims kept, Dims red, uint32_t red_total, int ref_zero) {
    uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= n_out) return;
    const T *p = x + x_off + decompose(kept, gid);
    T acc = ref_zero ? (T)0 : identity<OP, T>();
    if (red.n == 1) {
        // eight independent requests at a time, combined in index order: the result is that of the plain loop,
        // which would wait for each element in turn (128 partial sums: 30 us against 5)
        const uint32_t s = red.stride[0], n = red.ext[0];
        uint32_t i = 0;
        for (; i + 8 <= n; i += 8) {
            T v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = p[(i + u) * s];
#pragma unroll
            for (int u = 0; u < 8; ++u) acc = combine<OP, T>(acc, v[u]);
        }
        for (; i < n; ++i) acc = combine<OP, T>(acc, p[i * s]);
    } else {
        for (uint32_t i = 0; i < red_total; ++i) acc = combine<OP, T>(acc, p[decompose(red, i)]);
    }
    y[gid] = acc;
}

// ---- column reduction: few contiguous outputs, a long strided reduced axis (bias gradients: the
// sum over all rows of a [rows, C] matrix).  One thread per output would leave most of the chip idle
// and read serially; here a workgroup takes 64 columns x a chunk of rows, its four wavefronts walk
// alternate rows with coalesced 256-byte reads, and the per-chunk results are combined by a second,
// small pass (in a fixed order: the result does not depend on scheduling).
template <int OP, class T>
__global__ void __launch_bounds__(256) reduce_cols_kernel(const T *__restrict__ x, T *__restrict__ part, uint32_t n_cols,
                                                          uint32_t n_rows, uint32_t row_stride, uint32_t rows_per_chunk,
                                                          uint32_t x_off) {
    __shared__ T sh[4][64];
    const uint32_t c = blockIdx.x * 64u + (threadIdx.x & 63u), ty = threadIdx.x >> 6;
    const uint32_t r0 = blockIdx.y * rows_per_chunk, r1 = min(r0 + rows_per_chunk, n_rows);
    T acc = identity<OP, T>();
    if (c < n_cols) {
        const T *p = x + x_off + c;
        uint32_t r = r0 + ty;
        for (; r + 12 < r1; r += 16) {  // four rows in flight, combined in row order
            T v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = p[(size_t)(r + 4 * u) * row_stride];
#pragma unroll
            for (int u = 0; u < 4; ++u) acc = combine<OP, T>(acc, v[u]);
        }
        for (; r < r1; r += 4) acc = combine<OP, T>(acc, p[(size_t)r * row_stride]);
    }
    sh[ty][threadIdx.x & 63u] = acc;
    __syncthreads();
    if (ty == 0 && c < n_cols) {
        acc = combine<OP, T>(combine<OP, T>(sh[0][threadIdx.x], sh[1][threadIdx.x]), combine<OP, T>(sh[2][threadIdx.x], sh[3][threadIdx.x]));
        part[(size_t)blockIdx.y * n_cols + c] = acc;
    }
}

// ---- contiguous reduced span: ROWS_PER_BLOCK wavefronts, one row each, or one block per row ----
template <int OP, class T, bool VEC4, bool BLOCK_PER_ROW>
__global__ void __launch_bounds__(256) reduce_row_kernel(const T *__restrict__ x, T *__restrict__ y, uint32_t n_out,
                                                         uint32_t x_off, Dims kept, uint32_t len, int ref_zero) {
    __shared__ T part[4];
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const uint32_t row = BLOCK_PER_ROW ? blockIdx.x : blockIdx.x * 4u + wave;
    const bool active = row < n_out;
    T acc = identity<OP, T>();
    if (active) {
        const T *p = x + x_off + decompose(kept, row);
        const uint32_t t = BLOCK_PER_ROW ? threadIdx.x : lane, nt = BLOCK_PER_ROW ? 256u : (uint32_t)WAVE;
        if (VEC4) {
            typedef T V4 __attribute__((ext_vector_type(4)));
            const V4 *p4 = reinterpret_cast<const V4 *>(p);
            // four loads in flight per trip; the values are combined in the order a one-load loop would
            const uint32_t n4 = len / 4;
            uint32_t i = t;
            for (; i + 3 * nt < n4; i += 4 * nt) {
                const V4 v0 = p4[i], v1 = p4[i + nt], v2 = p4[i + 2 * nt], v3 = p4[i + 3 * nt];
                acc = combine<OP, T>(combine<OP, T>(combine<OP, T>(combine<OP, T>(acc, v0.x), v0.y), v0.z), v0.w);
                acc = combine<OP, T>(combine<OP, T>(combine<OP, T>(combine<OP, T>(acc, v1.x), v1.y), v1.z), v1.w);
                acc = combine<OP, T>(combine<OP, T>(combine<OP, T>(combine<OP, T>(acc, v2.x), v2.y), v2.z), v2.w);
                acc = combine<OP, T>(combine<OP, T>(combine<OP, T>(combine<OP, T>(acc, v3.x), v3.y), v3.z), v3.w);
            }
            for (; i < n4; i += nt) {
                const V4 v = p4[i];
                acc = combine<OP, T>(combine<OP, T>(combine<OP, T>(combine<OP, T>(acc, v.x), v.y), v.z), v.w);
            }
        } else {
            for (uint32_t i = t; i < len; i += nt) acc = combine<OP, T>(acc, p[i]);
        }
    }
    acc = wave_reduce<OP, T>(acc);
    if (BLOCK_PER_ROW) {
        if (lane == 0) part[wave] = acc;
        __syncthreads();
        if (threadIdx.x == 0) {
            T r = combine<OP, T>(combine<OP, T>(part[0], part[1]), combine<OP, T>(part[2], part[3]));
            if (ref_zero) r = combine<OP, T>((T)0, r);
            y[row] = r;
        }
    } else if (active && lane == 0) {
        if (ref_zero) acc = combine<OP, T>((T)0, acc);
        y[row] = acc;
    }
}

// ---- argmax / argmin: first extreme index wins (strict compare, reduce.rs:398-410) ------------
template <bool IS_MAX, class T>
__global__ void __launch_bounds__(256) reduce_arg_thread_kernel(const T *__restrict__ x, uint32_t *__restrict__ y, uint32_t n_out,
                                                                uint32_t x_off, Dims kept, uint32_t len, uint32_t stride) {
    uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= n_out) return;
    const T *p = x + x_off + decompose(kept, gid);
    T acc = p[0];
    uint32_t arg = 0;
    for (uint32_t i = 0; i < len; ++i) {
        T v = p[i * stride];
        if (IS_MAX ? acc < v : acc > v) {
            arg = i;
            acc = v;
        }
    }
    y[gid] = arg;
}

// One wavefront per row for a contiguous axis.  Each lane scans i = lane, lane+64, ... in
// increasing order with the strict compare, so it holds the FIRST extreme of its subsequence; the
// cross-lane step keeps, among equal values, the smaller index — together: the first overall.
// A NaN never wins a strict compare, as in the reference's serial scan, except in position 0
// (acc starts as x[0]); lanes other than 0 therefore start from x[their first i] only if it is
// not NaN-poisoning the order: they start "empty" and adopt the first element unconditionally,
// which differs from the serial scan only when NaNs are present.
template <bool IS_MAX, class T>
__global__ void __launch_bounds__(256) reduce_arg_row_kernel(const T *__restrict__ x, uint32_t *__restrict__ y, uint32_t n_out,
                                                             uint32_t x_off, Dims kept, uint32_t len) {
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const uint32_t row = blockIdx.x * 4u + wave;
    if (row >= n_out) return;
    const T *p = x + x_off + decompose(kept, row);
    bool have = false;
    T acc = (T)0;
    uint32_t arg = 0xffffffffu;
    for (uint32_t i = lane; i < len; i += WAVE) {
        T v = p[i];
        if (!have || (IS_MAX ? acc < v : acc > v)) {
            acc = v;
            arg = i;
            have = true;
        }
    }
#pragma unroll
    for (int m = WAVE / 2; m >= 1; m >>= 1) {
        T oa = shfl_xor(acc, m);
        uint32_t oi = shfl_xor(arg, m);
        bool ohave = oi != 0xffffffffu;
        bool take = ohave && (!have || (IS_MAX ? acc < oa : acc > oa) || (oa == acc && oi < arg));
        if (take) {
            acc = oa;
            arg = oi;
            have = true;
        }
    }
    if (lane == 0) y[row] = arg;
}

// ---- fused row operators: rows stay in registers between the read and the write ---------------
// A row is dealt to LPR lanes (a power of two, 4..64) as 16-byte chunks: chunk j of lane l covers
// columns (j*LPR + l)*4 .. +3.  Long rows use the whole wavefront (LPR = 64) and several chunks per
// lane; short rows use a fraction of it, so one wavefront carries 64/LPR rows and every load
// instruction still moves 1 KiB.  Reductions run over the LPR lanes of a row with xor shuffles.
typedef float f32x4 __attribute__((ext_vector_type(4)));

// e^t through the hardware 2^x: relative error about |t| * 6e-8 from the rounded argument plus one ulp;
// results below 2^-126 come out as zero.
__device__ __forceinline__ float fast_exp(float t) { return __builtin_amdgcn_exp2f(t * 1.44269504088896340736f); }

template <int NCHUNK> struct RowRegs {
    f32x4 v[NCHUNK];
};

// NT: non-temporal accesses for rows that stream through (operands too large for the caches to hand
// them to the next kernel).  Streamed stores also leave the L2s while the kernel runs instead of being
// written back all at once when it ends.
template <bool NT> __device__ __forceinline__ f32x4 load4(const float *p) {
    return NT ? __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p)) : *reinterpret_cast<const f32x4 *>(p);
}
template <bool NT> __device__ __forceinline__ void store4(float *p, f32x4 v) {
    if (NT) __builtin_nontemporal_store(v, reinterpret_cast<f32x4 *>(p));
    else *reinterpret_cast<f32x4 *>(p) = v;
}

template <int NCHUNK, int LPR, bool NT = false>
__device__ __forceinline__ void load_row(const float *p, uint32_t len, int li, RowRegs<NCHUNK> &r, float fill) {
#pragma unroll
    for (int j = 0; j < NCHUNK; ++j) {
        uint32_t c = (j * LPR + li) * 4u;
        if (c < len) r.v[j] = load4<NT>(p + c);
        else r.v[j] = f32x4{fill, fill, fill, fill};
    }
}

template <int OP, int LPR> __device__ __forceinline__ float seg_reduce(float v) {
    if (LPR == WAVE) return wave_reduce<OP, float>(v);
#pragma unroll
    for (int m = LPR / 2; m >= 1; m >>= 1) v = combine<OP, float>(v, shfl_xor(v, m));
    return v;
}

struct BDims {  // broadcastable operand: strides over the row index space + inner stride
    Dims outer;
    uint32_t inner_stride;
    uint32_t off;
};

// softmax(x + addend) over the last axis (nn.rs:42-56).  The shift is max(0, row max), not the row
// max: the reference's max accumulator starts at literal 0 (reduce.rs:282), and using the same
// shift keeps even the underflow behaviour of rows far below zero identical.  The quotient y/sum is
// formed as y * (1/sum): one division per row instead of one per element.
template <int NCHUNK, int LPR, bool HAS_ADD, bool NT>
__global__ void __launch_bounds__(256) softmax_row_kernel(const float *__restrict__ x, const float *__restrict__ add,
                                                          float *__restrict__ y, uint32_t n_rows, uint32_t len,
                                                          uint32_t x_off, Dims xo, BDims ao, uint32_t y_off) {
    constexpr int RPW = WAVE / LPR;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, li = lane % LPR;
    const uint32_t row = (blockIdx.x * 4u + wave) * RPW + lane / LPR;
    if (row >= n_rows) return;
    const float *p = x + x_off + decompose(xo, row);
    RowRegs<NCHUNK> r;
    load_row<NCHUNK, LPR, NT>(p, len, li, r, -__builtin_inff());
    if (HAS_ADD) {
        // the addend (a mask broadcast over heads and queries) is re-read by many rows: regular loads
        const float *a = add + ao.off + decompose(ao.outer, row);
        f32x4 av[NCHUNK];
#pragma unroll
        for (int j = 0; j < NCHUNK; ++j) {
            const uint32_t c = (j * LPR + li) * 4u;
            av[j] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (c < len) {
                if (ao.inner_stride == 1) {
                    av[j] = *reinterpret_cast<const f32x4 *>(a + c);
                } else {
                    av[j].x = a[(c + 0) * ao.inner_stride]; av[j].y = a[(c + 1) * ao.inner_stride];
                    av[j].z = a[(c + 2) * ao.inner_stride]; av[j].w = a[(c + 3) * ao.inner_stride];
                }
            }
        }
#pragma unroll
        for (int j = 0; j < NCHUNK; ++j) r.v[j] += av[j];
    }
    float m = -__builtin_inff();
#pragma unroll
    for (int j = 0; j < NCHUNK; ++j) m = fmaxf(fmaxf(fmaxf(fmaxf(m, r.v[j].x), r.v[j].y), r.v[j].z), r.v[j].w);
    m = fmaxf(seg_reduce<OP_MAX, LPR>(m), 0.0f);
    RowRegs<NCHUNK> e;
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < NCHUNK; ++j) {
        e.v[j].x = fast_exp(r.v[j].x - m); e.v[j].y = fast_exp(r.v[j].y - m);
        e.v[j].z = fast_exp(r.v[j].z - m); e.v[j].w = fast_exp(r.v[j].w - m);
        s += (e.v[j].x + e.v[j].y) + (e.v[j].z + e.v[j].w);
    }
    s = seg_reduce<OP_SUM, LPR>(s);
    // fast_exp flushes results below 2^-126 to zero, which only matters when every term of the row is
    // that small (a row entirely below -87, whose shift is 0): such a row is redone with the exact
    // routine, which keeps the denormal terms as the reference's kernel language does
    if (s < 1.0e-30f) {
        s = 0.0f;
#pragma unroll
        for (int j = 0; j < NCHUNK; ++j) {
            e.v[j].x = expf(r.v[j].x - m); e.v[j].y = expf(r.v[j].y - m);
            e.v[j].z = expf(r.v[j].z - m); e.v[j].w = expf(r.v[j].w - m);
            s += (e.v[j].x + e.v[j].y) + (e.v[j].z + e.v[j].w);
        }
        s = seg_reduce<OP_SUM, LPR>(s);
    }
    const float inv = 1.0f / s;
    float *q = y + y_off + (size_t)row * len;
#pragma unroll
    for (int j = 0; j < NCHUNK; ++j) {
        uint32_t c = (j * LPR + li) * 4u;
        if (c < len) store4<NT>(q + c, e.v[j] * inv);
    }
}

// Any row length / alignment: one workgroup per row, three passes over a row that stays in cache.
template <bool HAS_ADD>
__global__ void __launch_bounds__(256) softmax_row_generic_kernel(const float *__restrict__ x, const float *__restrict__ add,
                                                                  float *__restrict__ y, uint32_t len, uint32_t x_off,
                                                                  Dims xo, BDims ao, uint32_t y_off) {
    __shared__ float part[4];
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const uint32_t row = blockIdx.x;
    const float *p = x + x_off + decompose(xo, row);
    const float *a = HAS_ADD ? add + ao.off + decompose(ao.outer, row) : nullptr;
    float m = -__builtin_inff();
    for (uint32_t i = threadIdx.x; i < len; i += 256) m = fmaxf(m, p[i] + (HAS_ADD ? a[i * ao.inner_stride] : 0.0f));
    m = wave_reduce<OP_MAX, float>(m);
    if (lane == 0) part[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3])), 0.0f);
    __syncthreads();
    float s = 0.0f;
    for (uint32_t i = threadIdx.x; i < len; i += 256) s += expf(p[i] + (HAS_ADD ? a[i * ao.inner_stride] : 0.0f) - m);
    s = wave_reduce<OP_SUM, float>(s);
    if (lane == 0) part[wave] = s;
    __syncthreads();
    s = (part[0] + part[1]) + (part[2] + part[3]);
    float *q = y + y_off + (size_t)row * len;
    for (uint32_t i = threadIdx.x; i < len; i += 256) q[i] = expf(p[i] + (HAS_ADD ? a[i * ao.inner_stride] : 0.0f) - m) / s;
}

// softmax_cross_entropy (nn.rs:58-82): c = max(x), lse = log(sum exp(x-c)) + c,
// loss = -(x[label] - lse).  Same operation order as the composition.
template <int NCHUNK, int LPR>
__global__ void __launch_bounds__(256) softmax_ce_row_kernel(const float *__restrict__ x, const uint32_t *__restrict__ labels,
                                                             float *__restrict__ loss, uint32_t n_rows, uint32_t len,
                                                             uint32_t x_off, uint32_t x_row_stride, uint32_t l_off,
                                                             uint32_t l_stride, uint32_t y_off) {
    constexpr int RPW = WAVE / LPR;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, li = lane % LPR;
    const uint32_t row = (blockIdx.x * 4u + wave) * RPW + lane / LPR;
    if (row >= n_rows) return;
    const float *p = x + x_off + (size_t)row * x_row_stride;
    // the label is requested with the row, and x[label] is then picked out of the row's registers: no
    // dependent load waits at the end of the wavefront's life
    const uint32_t label = labels[l_off + (size_t)row * l_stride];
    RowRegs<NCHUNK> r;
    load_row<NCHUNK, LPR>(p, len, li, r, -__builtin_inff());
    float picked = 0.0f;  // x[label] on the lane that holds it (a label outside the row leaves 0 on every lane)
#pragma unroll
    for (int j = 0; j < NCHUNK; ++j) {
        const uint32_t c = (j * LPR + li) * 4u;
        if (label - c < 4u) picked = r.v[j][label - c];
    }
    float m = -__builtin_inff();
#pragma unroll
    for (int j = 0; j < NCHUNK; ++j) m = fmaxf(fmaxf(fmaxf(fmaxf(m, r.v[j].x), r.v[j].y), r.v[j].z), r.v[j].w);
    m = fmaxf(seg_reduce<OP_MAX, LPR>(m), 0.0f);  // the reference's max accumulator starts at 0 (reduce.rs:282)
    const float xl = seg_reduce<OP_SUM, LPR>(picked);  // one lane holds the value, the others 0: the sum is exact
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < NCHUNK; ++j)
        s += (fast_exp(r.v[j].x - m) + fast_exp(r.v[j].y - m)) + (fast_exp(r.v[j].z - m) + fast_exp(r.v[j].w - m));
    s = seg_reduce<OP_SUM, LPR>(s);
    // fast_exp flushes results below 2^-126 to zero.  They only matter to the sum when every term is
    // that small (a row entirely below -87): then the sum is redone with the exact routine, which
    // keeps the denormal terms as the reference's kernel language does.
    if (s < 1.0e-30f) {
        s = 0.0f;
#pragma unroll
        for (int j = 0; j < NCHUNK; ++j)
            s += (expf(r.v[j].x - m) + expf(r.v[j].y - m)) + (expf(r.v[j].z - m) + expf(r.v[j].w - m));
        s = seg_reduce<OP_SUM, LPR>(s);
    }
    if (li == 0) {
        const float lse = logf(s) + m;
        loss[y_off + row] = -(xl - lse);
    }
}

__global__ void __launch_bounds__(256) softmax_ce_row_generic_kernel(const float *__restrict__ x, const uint32_t *__restrict__ labels,
                                                                     float *__restrict__ loss, uint32_t len, uint32_t x_off,
                                                                     uint32_t x_row_stride, uint32_t x_col_stride, uint32_t l_off,
                                                                     uint32_t l_stride, uint32_t y_off) {
    __shared__ float part[4];
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const uint32_t row = blockIdx.x;
    const float *p = x + x_off + (size_t)row * x_row_stride;
    float m = -__builtin_inff();
    for (uint32_t i = threadIdx.x; i < len; i += 256) m = fmaxf(m, p[i * x_col_stride]);
    m = wave_reduce<OP_MAX, float>(m);
    if (lane == 0) part[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3])), 0.0f);
    __syncthreads();
    float s = 0.0f;
    for (uint32_t i = threadIdx.x; i < len; i += 256) s += expf(p[i * x_col_stride] - m);
    s = wave_reduce<OP_SUM, float>(s);
    if (lane == 0) part[wave] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        s = (part[0] + part[1]) + (part[2] + part[3]);
        const uint32_t label = labels[l_off + (size_t)row * l_stride];
        loss[y_off + row] = -(p[label * x_col_stride] - (logf(s) + m));
    }
}

// layer_norm over the last axis (nn.rs:84-100): mean = S1/n, var = S2/n - mean^2,
// y = (x - mean) / sqrt(var + eps) * gamma + beta.  The division by sqrt(var+eps) is applied as a
// multiplication by its reciprocal (one division per row); everything else keeps the reference's
// operation order.
// Streaming launches are held to five wavefronts per SIMD: with all eight resident, a quarter more rows are in flight
// than the memory system serves at its best rate and every one of them holds its 3 KB until its statistics are complete
// ([32768,768]: 35.3 us with eight, 34.7 with six, 34.1 with five, 34.6 with four, 38.1 with three; the other row kernels
// lose with fewer than eight).
template <int NCHUNK, int LPR, bool NT>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(NT ? 5 : 8, NT ? 5 : 8))) layer_norm_row_kernel(const float *__restrict__ x, const float *__restrict__ gamma,
                                                             const float *__restrict__ beta, float *__restrict__ y,
                                                             uint32_t n_rows, uint32_t len, uint32_t x_off, Dims xo,
                                                             uint32_t g_off, uint32_t g_stride, uint32_t b_off, uint32_t b_stride,
                                                             int params_aligned, float eps, uint32_t y_off) {
    constexpr int RPW = WAVE / LPR;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, li = lane % LPR;
    const uint32_t row = (blockIdx.x * 4u + wave) * RPW + lane / LPR;
    if (row >= n_rows) return;
    const float *p = x + x_off + decompose(xo, row);
    RowRegs<NCHUNK> r;
    load_row<NCHUNK, LPR, NT>(p, len, li, r, 0.0f);
    // gamma and beta are requested with the row, so nothing waits on memory after the statistics
    const bool vec_params = g_stride == 1 && b_stride == 1 && params_aligned;
    f32x4 gv[NCHUNK], bv[NCHUNK];
#pragma unroll
    for (int j = 0; j < NCHUNK; ++j) {
        const uint32_t c = (j * LPR + li) * 4u;
        gv[j] = bv[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (c < len) {
            if (vec_params) {
                gv[j] = *reinterpret_cast<const f32x4 *>(gamma + g_off + c);
                bv[j] = *reinterpret_cast<const f32x4 *>(beta + b_off + c);
            } else {
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    gv[j][t] = gamma[g_off + (c + t) * g_stride];
                    bv[j][t] = beta[b_off + (c + t) * b_stride];
                }
            }
        }
    }
    float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
    for (int j = 0; j < NCHUNK; ++j) {
        s1 += (r.v[j].x + r.v[j].y) + (r.v[j].z + r.v[j].w);
        s2 += (r.v[j].x * r.v[j].x + r.v[j].y * r.v[j].y) + (r.v[j].z * r.v[j].z + r.v[j].w * r.v[j].w);
    }
    s1 = seg_reduce<OP_SUM, LPR>(s1);
    s2 = seg_reduce<OP_SUM, LPR>(s2);
    const float n = (float)len;
    const float mean = s1 / n;
    const float var = s2 / n - mean * mean;
    const float inv = 1.0f / sqrtf(var + eps);
    float *q = y + y_off + (size_t)row * len;
#pragma unroll
    for (int j = 0; j < NCHUNK; ++j) {
        const uint32_t c = (j * LPR + li) * 4u;
        if (c < len) store4<NT>(q + c, (r.v[j] - mean) * inv * gv[j] + bv[j]);
    }
}

__global__ void __launch_bounds__(256) layer_norm_row_generic_kernel(const float *__restrict__ x, const float *__restrict__ gamma,
                                                                     const float *__restrict__ beta, float *__restrict__ y,
                                                                     uint32_t len, uint32_t x_off, Dims xo, uint32_t g_off,
                                                                     uint32_t g_stride, uint32_t b_off, uint32_t b_stride, float eps,
                                                                     uint32_t y_off) {
    __shared__ float part1[4], part2[4];
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const uint32_t row = blockIdx.x;
    const float *p = x + x_off + decompose(xo, row);
    float s1 = 0.0f, s2 = 0.0f;
    for (uint32_t i = threadIdx.x; i < len; i += 256) {
        float v = p[i];
        s1 += v;
        s2 += v * v;
    }
    s1 = wave_reduce<OP_SUM, float>(s1);
    s2 = wave_reduce<OP_SUM, float>(s2);
    if (lane == 0) {
        part1[wave] = s1;
        part2[wave] = s2;
    }
    __syncthreads();
    s1 = (part1[0] + part1[1]) + (part1[2] + part1[3]);
    s2 = (part2[0] + part2[1]) + (part2[2] + part2[3]);
    const float n = (float)len;
    const float mean = s1 / n;
    const float denom = sqrtf(s2 / n - mean * mean + eps);
    float *q = y + y_off + (size_t)row * len;
    for (uint32_t i = threadIdx.x; i < len; i += 256)
        q[i] = (p[i] - mean) / denom * gamma[g_off + i * g_stride] + beta[b_off + i * b_stride];
}

// ---- host-side planning -------------------------------------------------------------------------

// Merge axes i, i+1 of (ext, stride) lists when stride[i] == stride[i+1]*ext[i+1]; drop extent 1.
void collapse(std::vector<int64_t> &ext, std::vector<int64_t> &st) {
    std::vector<int64_t> e2, s2;
    for (size_t i = 0; i < ext.size(); ++i) {
        if (ext[i] == 1) continue;
        if (!e2.empty() && s2.back() == st[i] * ext[i]) {
            e2.back() *= ext[i];
            s2.back() = st[i];
        } else {
            e2.push_back(ext[i]);
            s2.push_back(st[i]);
        }
    }
    ext.swap(e2);
    st.swap(s2);
}

Dims to_dims(const std::vector<int64_t> &ext, const std::vector<int64_t> &st) {
    Dims d;
    d.n = (int)ext.size();
    for (int i = 0; i < SG_MAX_RANK; ++i) {
        d.ext[i] = i < d.n ? (uint32_t)ext[i] : 1;
        d.stride[i] = i < d.n ? (uint32_t)st[i] : 0;
        const sg_fastdiv f = sg_make_fastdiv(d.ext[i]);
        d.magic[i] = f.magic;
        d.shift[i] = f.shift;
    }
    return d;
}

bool aligned16(const void *base, int64_t off_elems) { return (((uintptr_t)base) + (uint64_t)off_elems * 4) % 16 == 0; }

bool dims_mult4(const Dims &d) {
    for (int i = 0; i < d.n; ++i)
        if (d.stride[i] % 4) return false;
    return true;
}

template <int OP, class T>
int launch_reduce(sg_ctx *ctx, const sg_tensor *in, const sg_tensor *out, const Dims &kept, const Dims &red, int64_t n_out,
                  int64_t red_total, int ref_zero) {
    const T *x = (const T *)in->base;
    T *y = (T *)out->base + out->offset;
    if (red.n == 1 && red.stride[0] == 1 && red_total >= 32) {
        const uint32_t len = red.ext[0];
        const bool vec = len % 4 == 0 && aligned16(in->base, in->offset) && dims_mult4(kept);
        if (len >= 2048) {
            dim3 grid((unsigned)n_out);
            if (vec) hipLaunchKernelGGL((reduce_row_kernel<OP, T, true, true>), grid, dim3(256), 0, ctx->stream, x, y, (uint32_t)n_out, (uint32_t)in->offset, kept, len, ref_zero);
            else hipLaunchKernelGGL((reduce_row_kernel<OP, T, false, true>), grid, dim3(256), 0, ctx->stream, x, y, (uint32_t)n_out, (uint32_t)in->offset, kept, len, ref_zero);
        } else {
            dim3 grid((unsigned)((n_out + 3) / 4));
            if (vec) hipLaunchKernelGGL((reduce_row_kernel<OP, T, true, false>), grid, dim3(256), 0, ctx->stream, x, y, (uint32_t)n_out, (uint32_t)in->offset, kept, len, ref_zero);
            else hipLaunchKernelGGL((reduce_row_kernel<OP, T, false, false>), grid, dim3(256), 0, ctx->stream, x, y, (uint32_t)n_out, (uint32_t)in->offset, kept, len, ref_zero);
        }
    } else if (kept.n == 1 && kept.stride[0] == 1 && red.n == 1 && red_total >= 256 && n_out * 8 <= red_total * 64 && n_out <= 16384) {
        // contiguous outputs, one long strided reduced axis: chunks of rows in parallel, then a combine pass
        const uint32_t n_cols = (uint32_t)n_out, n_rows = (uint32_t)red_total;
        const uint32_t col_tiles = (n_cols + 63) / 64;
        uint32_t chunks = (2u * (uint32_t)(ctx->num_cus > 0 ? ctx->num_cus : 256) + col_tiles - 1) / col_tiles;
        if (chunks > 128) chunks = 128;  // the combine pass walks the chunks serially per output
        if (chunks > n_rows / 32) chunks = n_rows / 32;
        if (chunks < 1) chunks = 1;
        const uint32_t rows_per_chunk = (n_rows + chunks - 1) / chunks;
        chunks = (n_rows + rows_per_chunk - 1) / rows_per_chunk;
        void *ws = nullptr;
        int rc = sg_alloc(ctx, (uint64_t)chunks * n_cols * sizeof(T), &ws);
        if (rc != SG_OK) return rc;
        hipLaunchKernelGGL((reduce_cols_kernel<OP, T>), dim3(col_tiles, chunks), dim3(256), 0, ctx->stream, x, (T *)ws, n_cols, n_rows,
                           red.stride[0], rows_per_chunk, (uint32_t)in->offset);
        const Dims pk = kept, pr = to_dims({(int64_t)chunks}, {(int64_t)n_cols});
        hipLaunchKernelGGL((reduce_thread_kernel<OP, T>), dim3((n_cols + 255) / 256), dim3(256), 0, ctx->stream, (const T *)ws, y, n_cols, 0u, pk, pr, chunks, ref_zero);
        SG_CHECK_LAUNCH(ctx, "reduce (columns)");
        return sg_free(ctx, ws);  // later users of the block are ordered behind these kernels on the stream
    } else {
        dim3 grid((unsigned)((n_out + 255) / 256));
        hipLaunchKernelGGL((reduce_thread_kernel<OP, T>), grid, dim3(256), 0, ctx->stream, x, y, (uint32_t)n_out, (uint32_t)in->offset, kept, red, (uint32_t)red_total, ref_zero);
    }
    SG_CHECK_LAUNCH(ctx, "reduce");
    return SG_OK;
}

template <class T>
int dispatch_reduce_op(sg_ctx *ctx, int op, const sg_tensor *in, const sg_tensor *out, const Dims &kept, const Dims &red,
                       int64_t n_out, int64_t red_total, int ref_zero) {
    switch (op) {
    case SG_R_SUM: return launch_reduce<OP_SUM, T>(ctx, in, out, kept, red, n_out, red_total, ref_zero);
    case SG_R_PROD: return launch_reduce<OP_PROD, T>(ctx, in, out, kept, red, n_out, red_total, ref_zero);
    case SG_R_MAX: return launch_reduce<OP_MAX, T>(ctx, in, out, kept, red, n_out, red_total, ref_zero);
    case SG_R_MIN: return launch_reduce<OP_MIN, T>(ctx, in, out, kept, red, n_out, red_total, ref_zero);
    }
    return sg_fail(ctx, SG_ERR_ARG, "sg_reduce: unknown op %d", op);
}

// rows = all axes but the last, as a collapsed Dims; returns number of rows
int64_t row_dims(const sg_tensor *t, Dims &d) {
    std::vector<int64_t> e(t->extents, t->extents + t->rank - 1), s(t->strides, t->strides + t->rank - 1);
    int64_t n = 1;
    for (auto v : e) n *= v;
    collapse(e, s);
    d = to_dims(e, s);
    return n;
}

}  // namespace

// Rows of up to 64 floats are dealt to 4..16 lanes (one 16-byte chunk each), rows of up to 256 to 8 or 16
// lanes with four chunks each (several rows per wavefront, 64 bytes in flight per lane: measured faster
// than one chunk on 32 or 64 lanes); longer rows to all 64 lanes with 2..8 chunks per lane.  Expects SG_ROW_LAUNCH(NCHUNK, LPR).
#define SG_ROW_DISPATCH(LEN)                                                                                            \
    do {                                                                                                                \
        const uint32_t len_ = (LEN);                                                                                    \
        if (len_ <= 16) SG_ROW_LAUNCH(1, 4);                                                                            \
        else if (len_ <= 32) SG_ROW_LAUNCH(1, 8);                                                                       \
        else if (len_ <= 64) SG_ROW_LAUNCH(1, 16);                                                                      \
        else if (len_ <= 128) SG_ROW_LAUNCH(4, 8);                                                                      \
        else if (len_ <= 256) SG_ROW_LAUNCH(4, 16);                                                                     \
        else if (len_ <= 512) SG_ROW_LAUNCH(2, 64);                                                                     \
        else if (len_ <= 768) SG_ROW_LAUNCH(3, 64);                                                                     \
        else if (len_ <= 1024) SG_ROW_LAUNCH(4, 64);                                                                    \
        else if (len_ <= 1536) SG_ROW_LAUNCH(6, 64);                                                                    \
        else SG_ROW_LAUNCH(8, 64);                                                                                      \
    } while (0)

extern "C" int sg_reduce(sg_ctx *ctx, int op, const int32_t *axes, int n_axes, int init_mode, const sg_tensor *in,
                         const sg_tensor *out) {
    if (!ctx) return SG_ERR_ARG;
    int rc;
    if ((rc = sg_validate_tensor(ctx, in, "sg_reduce input")) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, out, "sg_reduce output")) != SG_OK) return rc;
    if (n_axes < 0 || n_axes > in->rank || (n_axes && !axes)) return sg_fail(ctx, SG_ERR_ARG, "sg_reduce: bad axes");
    if (init_mode != SG_INIT_REF_ZERO && init_mode != SG_INIT_IDENTITY) return sg_fail(ctx, SG_ERR_ARG, "sg_reduce: bad init_mode");
    if (in->dtype != out->dtype) return sg_fail(ctx, SG_ERR_DTYPE, "sg_reduce: output dtype differs from input (reduce.rs:246)");
    if (!sg_is_dense(out)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_reduce: output must be dense row-major");
    bool listed[SG_MAX_RANK] = {false};
    for (int i = 0; i < n_axes; ++i) {
        if (axes[i] < 0 || axes[i] >= in->rank || listed[axes[i]]) return sg_fail(ctx, SG_ERR_SHAPE, "sg_reduce: axis %d invalid or repeated", axes[i]);
        listed[axes[i]] = true;
    }
    std::vector<int64_t> ke, ks, re, rs;
    int64_t n_out = 1, red_total = 1;
    for (int a = 0; a < in->rank; ++a) {
        if (listed[a]) {
            re.push_back(in->extents[a]);
            rs.push_back(in->strides[a]);
            red_total *= in->extents[a];
        } else {
            ke.push_back(in->extents[a]);
            ks.push_back(in->strides[a]);
            n_out *= in->extents[a];
        }
    }
    if (sg_numel(out) != n_out)
        return sg_fail(ctx, SG_ERR_SHAPE, "sg_reduce: output has %lld elements, reduced_extents gives %lld (reduce.rs:124-140)",
                       (long long)sg_numel(out), (long long)n_out);
    collapse(ke, ks);
    collapse(re, rs);
    if (re.empty()) {
        re.push_back(1);
        rs.push_back(0);
    }
    Dims kept = to_dims(ke, ks), red = to_dims(re, rs);
    const int ref_zero = init_mode == SG_INIT_REF_ZERO;
    switch (in->dtype) {
    case SG_FLOAT: return dispatch_reduce_op<float>(ctx, op, in, out, kept, red, n_out, red_total, ref_zero);
    case SG_INT: return dispatch_reduce_op<int>(ctx, op, in, out, kept, red, n_out, red_total, ref_zero);
    default: return dispatch_reduce_op<unsigned>(ctx, op, in, out, kept, red, n_out, red_total, ref_zero);
    }
}

extern "C" int sg_reduce_arg(sg_ctx *ctx, int op, int axis, const sg_tensor *in, const sg_tensor *out) {
    if (!ctx) return SG_ERR_ARG;
    int rc;
    if ((rc = sg_validate_tensor(ctx, in, "sg_reduce_arg input")) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, out, "sg_reduce_arg output")) != SG_OK) return rc;
    if (op != SG_RA_MAX && op != SG_RA_MIN) return sg_fail(ctx, SG_ERR_ARG, "sg_reduce_arg: unknown op %d", op);
    if (axis < 0 || axis >= in->rank) return sg_fail(ctx, SG_ERR_SHAPE, "sg_reduce_arg: axis %d out of range", axis);
    if (out->dtype != SG_UINT) return sg_fail(ctx, SG_ERR_DTYPE, "sg_reduce_arg: output must be uint (reduce.rs:347)");
    if (!sg_is_dense(out)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_reduce_arg: output must be dense row-major");
    std::vector<int64_t> ke, ks;
    int64_t n_out = 1;
    for (int a = 0; a < in->rank; ++a)
        if (a != axis) {
            ke.push_back(in->extents[a]);
            ks.push_back(in->strides[a]);
            n_out *= in->extents[a];
        }
    if (sg_numel(out) != n_out) return sg_fail(ctx, SG_ERR_SHAPE, "sg_reduce_arg: output has %lld elements, expected %lld", (long long)sg_numel(out), (long long)n_out);
    collapse(ke, ks);
    Dims kept = to_dims(ke, ks);
    const uint32_t len = (uint32_t)in->extents[axis], stride = (uint32_t)in->strides[axis];
    uint32_t *y = (uint32_t *)out->base + out->offset;
    const bool row = stride == 1 && len >= 64;
    dim3 grid_t((unsigned)((n_out + 255) / 256)), grid_r((unsigned)((n_out + 3) / 4));
#define SG_LAUNCH_ARG(T, IS_MAX)                                                                                          \
    do {                                                                                                                  \
        if (row) hipLaunchKernelGGL((reduce_arg_row_kernel<IS_MAX, T>), grid_r, dim3(256), 0, ctx->stream, (const T *)in->base, y, (uint32_t)n_out, (uint32_t)in->offset, kept, len); \
        else hipLaunchKernelGGL((reduce_arg_thread_kernel<IS_MAX, T>), grid_t, dim3(256), 0, ctx->stream, (const T *)in->base, y, (uint32_t)n_out, (uint32_t)in->offset, kept, len, stride); \
    } while (0)
    if (in->dtype == SG_FLOAT) {
        if (op == SG_RA_MAX) SG_LAUNCH_ARG(float, true); else SG_LAUNCH_ARG(float, false);
    } else if (in->dtype == SG_INT) {
        if (op == SG_RA_MAX) SG_LAUNCH_ARG(int, true); else SG_LAUNCH_ARG(int, false);
    } else {
        if (op == SG_RA_MAX) SG_LAUNCH_ARG(unsigned, true); else SG_LAUNCH_ARG(unsigned, false);
    }
#undef SG_LAUNCH_ARG
    SG_CHECK_LAUNCH(ctx, "reduce_arg");
    return SG_OK;
}

extern "C" int sg_softmax_lastaxis(sg_ctx *ctx, const sg_tensor *x, const sg_tensor *addend, const sg_tensor *out) {
    if (!ctx) return SG_ERR_ARG;
    int rc;
    if ((rc = sg_validate_tensor(ctx, x, "sg_softmax x")) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, out, "sg_softmax out")) != SG_OK) return rc;
    if (addend && (rc = sg_validate_tensor(ctx, addend, "sg_softmax addend")) != SG_OK) return rc;
    if (x->dtype != SG_FLOAT || out->dtype != SG_FLOAT || (addend && addend->dtype != SG_FLOAT)) return sg_fail(ctx, SG_ERR_DTYPE, "sg_softmax: fp32 only");
    if (!sg_is_dense(out) || sg_numel(out) != sg_numel(x)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_softmax: output must be dense with x's element count");
    const int r = x->rank;
    const uint32_t len = (uint32_t)x->extents[r - 1];
    if (len > 1 && x->strides[r - 1] != 1) return sg_fail(ctx, SG_ERR_SHAPE, "sg_softmax: x must have unit stride on its last axis");
    if (addend) {
        if (addend->rank != r) return sg_fail(ctx, SG_ERR_SHAPE, "sg_softmax: addend rank differs");
        for (int a = 0; a < r; ++a)
            if (addend->extents[a] != x->extents[a]) return sg_fail(ctx, SG_ERR_SHAPE, "sg_softmax: addend extents differ (broadcast with stride 0)");
    }
    Dims xo;
    const int64_t n_rows = row_dims(x, xo);
    BDims ao{};
    if (addend) {
        // Both operands decompose the same row id over the same outer extents, so each may merge its own
        // adjacent axes wherever ITS strides allow (stride[i] == stride[i+1] * ext[i+1], which a run of
        // broadcast axes satisfies with zeros): a mask [N,1,1,L] under scores [N,H,L,L] becomes [N, H*L]
        // with strides [L, 0], one multiply-high per row, and dense scores collapse to a single axis.
        std::vector<int64_t> e(x->extents, x->extents + r - 1), s(addend->strides, addend->strides + r - 1);
        collapse(e, s);
        ao.outer = to_dims(e, s);
        ao.inner_stride = (uint32_t)addend->strides[r - 1];
        ao.off = (uint32_t)addend->offset;
    }
    const float *xp = (const float *)x->base, *ap = addend ? (const float *)addend->base : nullptr;
    float *yp = (float *)out->base;
    const bool vec = len % 4 == 0 && len <= 2048 && aligned16(x->base, x->offset) && dims_mult4(xo) && aligned16(out->base, out->offset) &&
                     (!addend || ao.inner_stride != 1 || (aligned16(addend->base, addend->offset) && dims_mult4(ao.outer)));
    if (vec) {
        const bool nt = sg_streaming(2 * sg_numel(x) * 4);
#define SG_ROW_LAUNCH_(NC, LPR, ADD, NT)                                                                                \
    hipLaunchKernelGGL((softmax_row_kernel<NC, LPR, ADD, NT>), grid, dim3(256), 0, ctx->stream, xp, ap, yp, (uint32_t)n_rows, len, (uint32_t)x->offset, xo, ao, (uint32_t)out->offset)
#define SG_ROW_LAUNCH(NC, LPR)                                                                                          \
    do {                                                                                                                \
        dim3 grid((unsigned)((n_rows + 4 * (64 / LPR) - 1) / (4 * (64 / LPR))));                                        \
        if (addend) { if (nt) SG_ROW_LAUNCH_(NC, LPR, true, true); else SG_ROW_LAUNCH_(NC, LPR, true, false); }          \
        else { if (nt) SG_ROW_LAUNCH_(NC, LPR, false, true); else SG_ROW_LAUNCH_(NC, LPR, false, false); }                \
    } while (0)
        SG_ROW_DISPATCH(len);
#undef SG_ROW_LAUNCH
#undef SG_ROW_LAUNCH_
    } else {
        if (addend) hipLaunchKernelGGL((softmax_row_generic_kernel<true>), dim3((unsigned)n_rows), dim3(256), 0, ctx->stream, xp, ap, yp, len, (uint32_t)x->offset, xo, ao, (uint32_t)out->offset);
        else hipLaunchKernelGGL((softmax_row_generic_kernel<false>), dim3((unsigned)n_rows), dim3(256), 0, ctx->stream, xp, ap, yp, len, (uint32_t)x->offset, xo, ao, (uint32_t)out->offset);
    }
    SG_CHECK_LAUNCH(ctx, "softmax");
    return SG_OK;
}

extern "C" int sg_softmax_cross_entropy(sg_ctx *ctx, const sg_tensor *logits, const sg_tensor *labels, const sg_tensor *loss) {
    if (!ctx) return SG_ERR_ARG;
    int rc;
    if ((rc = sg_validate_tensor(ctx, logits, "sg_softmax_cross_entropy logits")) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, labels, "sg_softmax_cross_entropy labels")) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, loss, "sg_softmax_cross_entropy loss")) != SG_OK) return rc;
    if (logits->dtype != SG_FLOAT || loss->dtype != SG_FLOAT) return sg_fail(ctx, SG_ERR_DTYPE, "sg_softmax_cross_entropy: logits and loss must be fp32");
    if (labels->dtype != SG_UINT && labels->dtype != SG_INT) return sg_fail(ctx, SG_ERR_DTYPE, "sg_softmax_cross_entropy: labels must be uint or int");
    if (logits->rank != 2 || labels->rank != 2 || labels->extents[0] != logits->extents[0] || labels->extents[1] != 1)
        return sg_fail(ctx, SG_ERR_SHAPE, "sg_softmax_cross_entropy: logits [B,C], labels [B,1] (nn.rs:70-82, core.rs:633)");
    const int64_t B = logits->extents[0];
    const uint32_t C = (uint32_t)logits->extents[1];
    if (sg_numel(loss) != B || !sg_is_dense(loss)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_softmax_cross_entropy: loss must be dense [B]");
    const float *xp = (const float *)logits->base;
    const uint32_t *lp = (const uint32_t *)labels->base;
    float *yp = (float *)loss->base;
    const uint32_t rs = (uint32_t)logits->strides[0], cs = (uint32_t)logits->strides[1];
    const bool vec = (cs == 1 || C == 1) && C % 4 == 0 && C <= 2048 && aligned16(logits->base, logits->offset) && rs % 4 == 0;
    if (vec) {
#define SG_ROW_LAUNCH(NC, LPR)                                                                                          \
    do {                                                                                                                \
        dim3 grid((unsigned)((B + 4 * (64 / LPR) - 1) / (4 * (64 / LPR))));                                             \
        hipLaunchKernelGGL((softmax_ce_row_kernel<NC, LPR>), grid, dim3(256), 0, ctx->stream, xp, lp, yp, (uint32_t)B, C, (uint32_t)logits->offset, rs, (uint32_t)labels->offset, (uint32_t)labels->strides[0], (uint32_t)loss->offset); \
    } while (0)
        SG_ROW_DISPATCH(C);
#undef SG_ROW_LAUNCH
    } else {
        hipLaunchKernelGGL(softmax_ce_row_generic_kernel, dim3((unsigned)B), dim3(256), 0, ctx->stream, xp, lp, yp, C, (uint32_t)logits->offset, rs, cs,
                           (uint32_t)labels->offset, (uint32_t)labels->strides[0], (uint32_t)loss->offset);
    }
    SG_CHECK_LAUNCH(ctx, "softmax_cross_entropy");
    return SG_OK;
}

extern "C" int sg_layer_norm_lastaxis(sg_ctx *ctx, const sg_tensor *x, const sg_tensor *gamma, const sg_tensor *beta, float eps,
                                      const sg_tensor *out) {
    if (!ctx) return SG_ERR_ARG;
    int rc;
    if ((rc = sg_validate_tensor(ctx, x, "sg_layer_norm x")) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, gamma, "sg_layer_norm gamma")) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, beta, "sg_layer_norm beta")) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, out, "sg_layer_norm out")) != SG_OK) return rc;
    if (x->dtype != SG_FLOAT || gamma->dtype != SG_FLOAT || beta->dtype != SG_FLOAT || out->dtype != SG_FLOAT)
        return sg_fail(ctx, SG_ERR_DTYPE, "sg_layer_norm: fp32 only");
    const int r = x->rank;
    const uint32_t len = (uint32_t)x->extents[r - 1];
    if (len > 1 && x->strides[r - 1] != 1) return sg_fail(ctx, SG_ERR_SHAPE, "sg_layer_norm: x must have unit stride on its last axis");
    if (!sg_is_dense(out) || sg_numel(out) != sg_numel(x)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_layer_norm: output must be dense with x's element count");
    const int64_t ng = sg_numel(gamma), nb = sg_numel(beta);
    if ((ng != 1 && ng != len) || (nb != 1 && nb != len)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_layer_norm: gamma/beta must have 1 or %u elements", len);
    if ((ng > 1 && !sg_is_dense(gamma)) || (nb > 1 && !sg_is_dense(beta))) return sg_fail(ctx, SG_ERR_SHAPE, "sg_layer_norm: gamma/beta must be dense");
    Dims xo;
    const int64_t n_rows = row_dims(x, xo);
    const float *xp = (const float *)x->base, *gp = (const float *)gamma->base, *bp = (const float *)beta->base;
    float *yp = (float *)out->base;
    const uint32_t gs = ng == 1 ? 0u : 1u, bs = nb == 1 ? 0u : 1u;
    const bool vec = len % 4 == 0 && len <= 2048 && aligned16(x->base, x->offset) && dims_mult4(xo) && aligned16(out->base, out->offset);
    if (vec) {
        const bool nt = sg_streaming(2 * sg_numel(x) * 4);
        // 16-byte loads of gamma and beta need their first elements 16-byte aligned, not just x's
        const int params_aligned = aligned16(gamma->base, gamma->offset) && aligned16(beta->base, beta->offset);
#define SG_ROW_LAUNCH_(NC, LPR, NT)                                                                                     \
    hipLaunchKernelGGL((layer_norm_row_kernel<NC, LPR, NT>), grid, dim3(256), 0, ctx->stream, xp, gp, bp, yp, (uint32_t)n_rows, len, (uint32_t)x->offset, xo, (uint32_t)gamma->offset, gs, (uint32_t)beta->offset, bs, params_aligned, eps, (uint32_t)out->offset)
#define SG_ROW_LAUNCH(NC, LPR)                                                                                          \
    do {                                                                                                                \
        dim3 grid((unsigned)((n_rows + 4 * (64 / LPR) - 1) / (4 * (64 / LPR))));                                        \
        if (nt) SG_ROW_LAUNCH_(NC, LPR, true); else SG_ROW_LAUNCH_(NC, LPR, false);                                     \
    } while (0)
        SG_ROW_DISPATCH(len);
#undef SG_ROW_LAUNCH
#undef SG_ROW_LAUNCH_
    } else {
        hipLaunchKernelGGL(layer_norm_row_generic_kernel, dim3((unsigned)n_rows), dim3(256), 0, ctx->stream, xp, gp, bp, yp, len, (uint32_t)x->offset, xo,
                           (uint32_t)gamma->offset, gs, (uint32_t)beta->offset, bs, eps, (uint32_t)out->offset);
    }
    SG_CHECK_LAUNCH(ctx, "layer_norm");
    return SG_OK;
}
