// Scaled-dot-product attention in one kernel, fp32 on the CDNA4 matrix cores, for gfx950.
//
// Replaces the operator chain of MultiHeadAttention::pass (bert.rs:262-271):
//   matmul_batched(q, k^T) -> div(sqrt(d)) -> add(extended mask) -> Softmax::pass(axis 3)
//   -> matmul_batched(., v) -> merge_heads copy
// i.e. two batched GEMMs (gemm.rs:53-104), two maps, the softmax composition of nn.rs:42-56 and an
// organize() copy, none of which keeps the [L,L] scores out of memory.
//
// Design:
//   * A workgroup of 4 wavefronts owns 128 queries of one (batch, head); a wavefront owns 32 of
//     them for the whole kernel.  Keys and values are walked in blocks of 64 through LDS.
//   * The score block is computed TRANSPOSED, S^T = K . Q^T (rows = keys, columns = queries), with
//     v_mfma_f32_32x32x2_f32.  In the accumulator layout a lane then holds one query (lane % 32)
//     and, in its 16 registers per 32-key block, the keys 8g + 4*(lane/32) + s (r = 4g + s).  That
//     is exactly the k assignment the next product needs for its B operand, so the probabilities
//     feed O^T = V^T . P^T straight from registers: no LDS round trip, no transposition.
//   * Softmax is online over key blocks (running shift m and sum l per query).  A query lives in two
//     lanes (l, l + 32), so the row statistics cost one cross-lane exchange.  The running shift
//     starts at 0 and only grows: the result uses the shift max(0, row max), as the reference's
//     softmax does (its max accumulator starts at literal 0, reduce.rs:282), including the 0/0 of a
//     fully masked row.
//   * O^T keeps the query in the lane as well, so rescaling by exp(m_old - m_new) and the final 1/l
//     are per-lane scalars, and the output leaves as 16-byte pieces of a query's row.
// Rounding differs from the reference's two-pass softmax and sequential-k products only at fp32
// rounding level (covered by the 1e-3 tolerance of GEMM-bearing paths).
#include "common.h"

#include <cstdlib>

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int NW = 4;          // wavefronts per workgroup
constexpr int KB = 64;         // keys per LDS block

struct AttnP {
    const float *q, *k, *v, *add;
    float *o;
    int Lq, Lk, nb1;
    int64_t q_sb0, q_sb1, q_sl, k_sb0, k_sb1, k_sl, v_sb0, v_sb1, v_sl, o_sb0, o_sb1, o_sl;
    int64_t a_sb0, a_sb1;  // addend strides over the two batch axes (0 = broadcast); per key, stride 1
    float scale;
    int vec_q, vec_k, vec_v, vec_o;
    int xcd_remap;  // workgroups of one (batch, head) on one XCD: they share its keys and values in that XCD's L2
    sg_fastdiv d_gx, d_nb1;  // division by gridDim.x and by nb1 as a multiply-high
};

// SPLIT = false: the four wavefronts take four groups of 32 queries and every wavefront walks all keys.
// SPLIT = true: the workgroup covers 64 queries; wavefronts 0,1 take the first 32 keys of every 64-key
// block and wavefronts 2,3 the other 32, and the two partial results of a query group are merged
// through LDS at the end (the exact merge of two online-softmax states).  Work units are half as
// large, which is what balances a short-sequence launch: B*H*L/32 units of 32 queries x all keys
// may come to 1.5 per SIMD (b32, 12 heads, s128: 1536 units on 1024 SIMDs), i.e. two rounds with half
// the chip idle in the second; split in two they are 3 per SIMD.  Three wavefronts per SIMD need the kernel
// within 168 registers (the compiler is told so below).  The unsplit kernel with one code path per load fits
// that limit too, but for three values spilled outside the key loop: a third workgroup per compute unit hides
// the others' prologues (430 -> 417 us at b64 x 12 heads x s512); with scalar fallbacks it stays at two.
//
// VEC = true: every operand row is 16-byte aligned, all global accesses are 16-byte ones and the code has no
// scalar fallbacks.  A launch starts with a cold instruction cache, and what a workgroup executes before its
// first MFMA is fetched line by line: at b32 x 12 heads x s128 the prologue (pointer arithmetic with two
// integer divisions, eight guarded and doubly coded Q loads, the first K/V requests) took 6 of the kernel's
// 22 us.  Hence: divisions by multiply-high, no guards (a query past the end computes on the last row and is
// not written; a key past the end reads as zeros through the buffer descriptor's range check and is masked
// with -inf), one code path per load, K and V requested through buffer loads with fixed per-lane offsets.
__device__ __forceinline__ uint32_t fdiv(uint32_t n, sg_fastdiv d) { return (__umulhi(n, d.magic) + n) >> d.shift; }

template <int D, bool SPLIT, bool VEC>
__global__ void __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu((SPLIT || VEC) ? 3 : 2, (SPLIT || VEC) ? 3 : 2))) attention_kernel(const AttnP p) {
    static_assert(D % 32 == 0 && D <= 64, "head size 32 or 64");
    constexpr int QB = SPLIT ? 64 : 32 * NW;   // queries per workgroup
    constexpr int NKB = SPLIT ? 1 : KB / 32;   // 32-key MFMA blocks a wavefront takes from an LDS block
    constexpr int LD = D + 4;              // LDS row stride (floats): 8 consecutive rows cover all banks
    constexpr int ND = D / 32;             // 32-wide blocks of the head dimension
    constexpr int NG = D / 8;              // groups of four k-steps over the head dimension
    constexpr int ROWV = D / 4;            // 16-byte pieces per K/V row
    constexpr int NLD = KB * ROWV / (64 * NW);  // 16-byte pieces of a K (or V) block per thread
    typedef float vecND __attribute__((ext_vector_type(ND)));  // one V value per output block of the head dimension
    __shared__ __attribute__((aligned(16))) float lds_k[KB * LD];
    __shared__ __attribute__((aligned(16))) float lds_v[KB * LD];
    __shared__ __attribute__((aligned(16))) float lds_m[KB];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ql = lane & 31, h = lane >> 5;
    // Workgroup ids go round-robin over the 8 XCDs.  Remapped, XCD x takes the x-th eighth of the (pair, query tile)
    // list, so the query tiles of one (batch, head) pair run on one XCD and fetch its keys and values into one L2.
    unsigned bx = blockIdx.x, by = blockIdx.y;
    if (p.xcd_remap) {
        const unsigned id = by * gridDim.x + bx, per = gridDim.x * gridDim.y / 8u;
        const unsigned nid = (id % 8u) * per + id / 8u;
        by = fdiv(nid, p.d_gx);
        bx = nid - by * gridDim.x;
    }
    const int bt0 = (int)fdiv(by, p.d_nb1), bt1 = (int)by - bt0 * p.nb1;
    const int q0 = bx * QB + (SPLIT ? (wave & 1) : wave) * 32;
    const int kw = SPLIT ? (wave >> 1) * 32 : 0;  // this wavefront's first key inside an LDS block
    const float *Q = p.q + bt0 * p.q_sb0 + bt1 * p.q_sb1;
    const float *K = p.k + bt0 * p.k_sb0 + bt1 * p.k_sb1;
    const float *V = p.v + bt0 * p.v_sb0 + bt1 * p.v_sb1;
    const float *A = p.add ? p.add + bt0 * p.a_sb0 + bt1 * p.a_sb1 : nullptr;

    // Q^T operand of this lane: Q[q][8g + 4h + s] for g < NG, s < 4 (filled below, through LDS)
    float qreg[NG][4];

    floatx16 oacc[ND];
#pragma unroll
    for (int j = 0; j < ND; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[j][r] = 0.0f;
    float m_run = 0.0f, l_run = 0.0f;  // shift (starts at the reference's 0) and this lane's share of the sum

    // global -> registers for one K/V block; piece f of the block: row f / ROWV, floats 4*(f % ROWV)..
    f32x4 kreg[NLD], vreg[NLD];
    float mreg = 0.0f;
    // VEC: the K and V requests are buffer loads: a descriptor per (batch, head) that ends behind the last key's row,
    // a per-lane byte offset fixed for the kernel (the piece's row and column inside a block) and a scalar offset per
    // block.  No address arithmetic on the vector unit in the key loop (it was a quarter of the loop's vector
    // instructions, and every one of them is paid in matrix-pipe cycles); a key past the end lies beyond the
    // descriptor's range and reads as zeros, its mask is -inf.
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    uint32_t koff[NLD], voff[NLD];
    __amdgpu_buffer_rsrc_t kdesc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(K), 0, 0, 0x00020000), vdesc = kdesc;
    if (VEC) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int f = tid + i * 64 * NW;
            const int row = f / ROWV, c = (f % ROWV) * 4;
            koff[i] = ((uint32_t)row * (uint32_t)p.k_sl + (uint32_t)c) * 4u;
            voff[i] = ((uint32_t)row * (uint32_t)p.v_sl + (uint32_t)c) * 4u;
        }
        kdesc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(K), 0, (int)(((uint32_t)(p.Lk - 1) * (uint32_t)p.k_sl + (uint32_t)D) * 4u), 0x00020000);
        vdesc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(V), 0, (int)(((uint32_t)(p.Lk - 1) * (uint32_t)p.v_sl + (uint32_t)D) * 4u), 0x00020000);
    }
    auto request = [&](int kb0) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            if (VEC) {
                kreg[i] = __builtin_bit_cast(f32x4, (u32x4)__builtin_amdgcn_raw_buffer_load_b128(kdesc, koff[i], (uint32_t)kb0 * (uint32_t)p.k_sl * 4u, 0));
                vreg[i] = __builtin_bit_cast(f32x4, (u32x4)__builtin_amdgcn_raw_buffer_load_b128(vdesc, voff[i], (uint32_t)kb0 * (uint32_t)p.v_sl * 4u, 0));
                continue;
            }
            const int f = tid + i * 64 * NW;
            const int row = f / ROWV, c = (f % ROWV) * 4;
            const int key = min(kb0 + row, p.Lk - 1);  // a key past the end repeats the last one (finite values); its mask is -inf
            const float *kp = K + (int64_t)key * p.k_sl + c, *vp = V + (int64_t)key * p.v_sl + c;
            f32x4 a, b;
            if (p.vec_k) a = *reinterpret_cast<const f32x4 *>(kp);
            else { a.x = kp[0]; a.y = kp[1]; a.z = kp[2]; a.w = kp[3]; }
            if (p.vec_v) b = *reinterpret_cast<const f32x4 *>(vp);
            else { b.x = vp[0]; b.y = vp[1]; b.z = vp[2]; b.w = vp[3]; }
            kreg[i] = a;
            vreg[i] = b;
        }
        if (tid < KB) {
            const int key = kb0 + tid;
            mreg = key < p.Lk ? (A ? A[key] : 0.0f) : -__builtin_inff();  // keys past the end never count
        }
    };
    auto deposit = [&]() {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int f = tid + i * 64 * NW;
            const int row = f / ROWV, c = (f % ROWV) * 4;
            *reinterpret_cast<f32x4 *>(&lds_k[row * LD + c]) = kreg[i];
            *reinterpret_cast<f32x4 *>(&lds_v[row * LD + c]) = vreg[i];
        }
        if (tid < KB) lds_m[tid] = mreg;
    };

    // The workgroup's Q tile goes through LDS: fetched like K and V (16 lanes per 256-byte row, whole cache lines),
    // then each lane picks its operand registers out of the tile.  Fetched straight into the operand layout, a load
    // instruction touches 32 rows for 32 bytes each, and with twelve wavefronts per compute unit doing so at once
    // the first-level cache's line rate, not memory, set the time (1.8 us of a 21 us kernel at b32 x 12 heads x s128).
    {
        constexpr int NQ = QB * ROWV / (64 * NW);
        f32x4 qtmp[NQ];
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            const int f = tid + i * 64 * NW;
            const int row = f / ROWV, c = (f % ROWV) * 4;
            const int q = min((int)bx * QB + row, p.Lq - 1);  // a query past the end repeats the last one; it is not written
            const float *src = Q + (int64_t)q * p.q_sl + c;
            if (VEC || p.vec_q) qtmp[i] = *reinterpret_cast<const f32x4 *>(src);
            else { qtmp[i].x = src[0]; qtmp[i].y = src[1]; qtmp[i].z = src[2]; qtmp[i].w = src[3]; }
        }
        request(0);  // the first K/V block is in flight behind the Q tile
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            const int f = tid + i * 64 * NW;
            const int row = f / ROWV, c = (f % ROWV) * 4;
            *reinterpret_cast<f32x4 *>(&(row < KB ? lds_k : lds_v)[(row % KB) * LD + c]) = qtmp[i];
        }
        __syncthreads();
        const int mine = (SPLIT ? (wave & 1) : wave) * 32 + ql;
        const float *src = &(mine < KB ? lds_k : lds_v)[(mine % KB) * LD + 4 * h];
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            const f32x4 t = *reinterpret_cast<const f32x4 *>(src + 8 * g);
            qreg[g][0] = t.x; qreg[g][1] = t.y; qreg[g][2] = t.z; qreg[g][3] = t.w;
        }
    }
    for (int kb0 = 0; kb0 < p.Lk; kb0 += KB) {
        __syncthreads();  // everyone is done reading the previous block
        deposit();
        __syncthreads();
        if (kb0 + KB < p.Lk) request(kb0 + KB);  // in flight during this block's arithmetic

        // ---- S^T block: keys x queries, contraction over the head dimension
        floatx16 sacc[NKB];
#pragma unroll
        for (int b = 0; b < NKB; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[b][r] = 0.0f;
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            f32x4 a[NKB];
#pragma unroll
            for (int b = 0; b < NKB; ++b) a[b] = *reinterpret_cast<const f32x4 *>(&lds_k[(kw + b * 32 + ql) * LD + 8 * g + 4 * h]);
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int b = 0; b < NKB; ++b) sacc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[b][s], qreg[g][s], sacc[b], 0, 0, 0);
        }

        // ---- scale, mask, online softmax.  Register r = 4g + s of block b is key 32b + 8g + 4h + s.
        float mloc = -__builtin_inff();
#pragma unroll
        for (int b = 0; b < NKB; ++b)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 mk = *reinterpret_cast<const f32x4 *>(&lds_m[kw + b * 32 + 8 * g + 4 * h]);
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const float x = sacc[b][4 * g + s] * p.scale + mk[s];
                    sacc[b][4 * g + s] = x;
                    mloc = fmaxf(mloc, x);
                }
            }
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
        const float m_new = fmaxf(m_run, mloc);
        // exp(x - m) as 2^(x*log2(e) - m*log2(e)): one fused multiply-add and the hardware exp2; the argument
        // rounding costs about |x - m| * 6e-8 relative, far inside the softmax tolerance
        constexpr float LOG2E = 1.44269504088896340736f;
        const float mshift = -m_new * LOG2E;
        // the shift rarely moves after the first blocks: when it stayed put for every query of the wavefront the
        // correction factor is exactly 1 and rescaling the accumulators (vector work the matrix pipe waits for) is skipped
        // (nothing to rescale in front of the first block: the accumulators and the sum are still zero)
        if (kb0 > 0 && __builtin_amdgcn_ballot_w64(m_new != m_run) != 0) {
            const float corr = __builtin_amdgcn_exp2f((m_run - m_new) * LOG2E);
            l_run *= corr;
#pragma unroll
            for (int j = 0; j < ND; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[j][r] *= corr;
        }
        m_run = m_new;
        float lsum = 0.0f;
#pragma unroll
        for (int b = 0; b < NKB; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[b][r], LOG2E, mshift));
                sacc[b][r] = e;
                lsum += e;
            }
        l_run += lsum;

        // ---- O^T += V^T . P^T: rows = head dimension, columns = queries, contraction over keys.
        // Row m of output block j stands for head index ND*m + j (any assignment of head indices to rows
        // works as long as the write-out agrees), so the ND values a lane feeds to the ND blocks for one
        // key are adjacent in the V row and come out of LDS as ONE read of 4*ND bytes.
#pragma unroll
        for (int b = 0; b < NKB; ++b)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                vecND a[4];
#pragma unroll
                for (int s = 0; s < 4; ++s) a[s] = *reinterpret_cast<const vecND *>(&lds_v[(kw + b * 32 + 8 * g + 4 * h + s) * LD + ND * ql]);
#pragma unroll
                for (int s = 0; s < 4; ++s)
#pragma unroll
                    for (int j = 0; j < ND; ++j) oacc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s][j], sacc[b][4 * g + s], oacc[j], 0, 0, 0);
            }
    }

    if (SPLIT) {
        // merge the two key halves of a query group: (m, l, O) of wavefront w + 2 into wavefront w, with
        // m = max(m_a, m_b), l = l_a e^(m_a - m) + l_b e^(m_b - m), O likewise; the K block's LDS is free now
        constexpr float LOG2E = 1.44269504088896340736f;
        constexpr int SLOT = 16 * ND + 2;  // floats per lane
        static_assert(2 * 64 * SLOT <= KB * LD, "the merge buffer fits in the K block");
        __syncthreads();
        if (wave >= 2) {
            float *dst = &lds_k[((wave - 2) * 64 + lane) * SLOT];
#pragma unroll
            for (int j = 0; j < ND; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) dst[16 * j + r] = oacc[j][r];
            dst[16 * ND] = m_run;
            dst[16 * ND + 1] = l_run;
        }
        __syncthreads();
        if (wave >= 2) return;
        const float *src = &lds_k[(wave * 64 + lane) * SLOT];
        const float m_b = src[16 * ND], l_b = src[16 * ND + 1];
        const float m = fmaxf(m_run, m_b);
        float ca = __builtin_amdgcn_exp2f((m_run - m) * LOG2E), cb = __builtin_amdgcn_exp2f((m_b - m) * LOG2E);
        l_run = l_run * ca + l_b * cb;
        // the 1/l of the normalisation below rides on the two merge factors: one multiplication per value less
        const float lm = l_run + __shfl_xor(l_run, 32, 64);
        const float invm = 1.0f / lm;
        ca *= invm;
        cb *= invm;
#pragma unroll
        for (int j = 0; j < ND; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[j][r] = oacc[j][r] * ca + src[16 * j + r] * cb;
    }
    // ---- normalise and write: register r = 4g + s of block j is head index ND*(8g + 4h + s) + j, so the
    // 4*ND values of one g are consecutive head indices starting at ND*(8g + 4h)
    const float l = l_run + __shfl_xor(l_run, 32, 64);
    const float inv = SPLIT ? 1.0f : 1.0f / l;
    const int q = q0 + ql;
    if (q < p.Lq) {
        float *row = p.o + bt0 * p.o_sb0 + bt1 * p.o_sb1 + (int64_t)q * p.o_sl;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float t[4 * ND];
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int j = 0; j < ND; ++j) t[ND * s + j] = oacc[j][4 * g + s] * inv;
            float *dst = row + ND * (8 * g + 4 * h);
#pragma unroll
            for (int c = 0; c < ND; ++c) {
                if (VEC || p.vec_o) *reinterpret_cast<f32x4 *>(dst + 4 * c) = f32x4{t[4 * c], t[4 * c + 1], t[4 * c + 2], t[4 * c + 3]};
                else { dst[4 * c] = t[4 * c]; dst[4 * c + 1] = t[4 * c + 1]; dst[4 * c + 2] = t[4 * c + 2]; dst[4 * c + 3] = t[4 * c + 3]; }
            }
        }
    }
}

bool aligned16(const void *base, int64_t offset_elems) { return ((uintptr_t)base + (uint64_t)offset_elems * 4) % 16 == 0; }

// [.., L, D] operand with up to two leading batch axes -> (pointer, batch strides, row stride)
int operand(sg_ctx *ctx, const sg_tensor *t, const char *who, int rank, const int64_t *batch, int64_t L, int64_t D, const float **ptr,
            int64_t *sb0, int64_t *sb1, int64_t *sl, int *vec) {
    int rc = sg_validate_tensor(ctx, t, who);
    if (rc != SG_OK) return rc;
    if (t->dtype != SG_FLOAT) return sg_fail(ctx, SG_ERR_DTYPE, "%s: fp32 only", who);
    if (t->rank != rank) return sg_fail(ctx, SG_ERR_SHAPE, "%s: rank %d, expected %d", who, t->rank, rank);
    for (int i = 0; i < rank - 2; ++i)
        if (t->extents[i] != batch[i]) return sg_fail(ctx, SG_ERR_SHAPE, "%s: batch extents differ", who);
    if (t->extents[rank - 2] != L || t->extents[rank - 1] != D) return sg_fail(ctx, SG_ERR_SHAPE, "%s: expected [.., %lld, %lld]", who, (long long)L, (long long)D);
    if (t->strides[rank - 1] != 1) return sg_fail(ctx, SG_ERR_SHAPE, "%s: the head dimension must have unit stride", who);
    *ptr = (const float *)t->base + t->offset;
    *sl = t->strides[rank - 2];
    *sb1 = rank >= 3 ? t->strides[rank - 3] : 0;
    *sb0 = rank >= 4 ? t->strides[rank - 4] : 0;
    *vec = aligned16(t->base, t->offset) && *sl % 4 == 0 && *sb0 % 4 == 0 && *sb1 % 4 == 0;
    return SG_OK;
}

}  // namespace

extern "C" int sg_attention(sg_ctx *ctx, const sg_tensor *q, const sg_tensor *k, const sg_tensor *v, const sg_tensor *addend, float scale,
                            const sg_tensor *out) {
    if (!ctx || !q || !k || !v || !out) return SG_ERR_ARG;
    const int rank = q->rank;
    if (rank < 2 || rank > 4) return sg_fail(ctx, SG_ERR_SHAPE, "sg_attention: rank 2..4");
    if (k->rank != rank) return sg_fail(ctx, SG_ERR_SHAPE, "sg_attention: k rank differs");
    const int64_t Lq = q->extents[rank - 2], D = q->extents[rank - 1], Lk = k->extents[rank - 2];
    if (D != 32 && D != 64) return sg_fail(ctx, SG_ERR_SHAPE, "sg_attention: head size %lld (32 and 64 are built)", (long long)D);
    if (Lq < 1 || Lk < 1) return sg_fail(ctx, SG_ERR_SHAPE, "sg_attention: empty sequence");
    int64_t batch[2] = {1, 1};
    for (int i = 0; i < rank - 2; ++i) batch[i] = q->extents[i];
    AttnP p{};
    int rc;
    const float *optr;
    if ((rc = operand(ctx, q, "sg_attention q", rank, batch, Lq, D, &p.q, &p.q_sb0, &p.q_sb1, &p.q_sl, &p.vec_q)) != SG_OK) return rc;
    if ((rc = operand(ctx, k, "sg_attention k", rank, batch, Lk, D, &p.k, &p.k_sb0, &p.k_sb1, &p.k_sl, &p.vec_k)) != SG_OK) return rc;
    if ((rc = operand(ctx, v, "sg_attention v", rank, batch, Lk, D, &p.v, &p.v_sb0, &p.v_sb1, &p.v_sl, &p.vec_v)) != SG_OK) return rc;
    if ((rc = operand(ctx, out, "sg_attention out", rank, batch, Lq, D, &optr, &p.o_sb0, &p.o_sb1, &p.o_sl, &p.vec_o)) != SG_OK) return rc;
    p.o = const_cast<float *>(optr);
    int64_t nb0 = 1, nb1 = 1;
    if (rank == 3) nb1 = batch[0];
    if (rank == 4) { nb0 = batch[0]; nb1 = batch[1]; }
    if (addend) {
        if ((rc = sg_validate_tensor(ctx, addend, "sg_attention addend")) != SG_OK) return rc;
        if (addend->dtype != SG_FLOAT) return sg_fail(ctx, SG_ERR_DTYPE, "sg_attention addend: fp32 only");
        if (addend->rank != rank) return sg_fail(ctx, SG_ERR_SHAPE, "sg_attention addend: rank differs");
        for (int i = 0; i < rank - 2; ++i)
            if (addend->extents[i] != batch[i]) return sg_fail(ctx, SG_ERR_SHAPE, "sg_attention addend: batch extents differ (broadcast with stride 0)");
        if (addend->extents[rank - 2] != Lq || addend->extents[rank - 1] != Lk) return sg_fail(ctx, SG_ERR_SHAPE, "sg_attention addend: expected [.., Lq, Lk]");
        if ((Lq > 1 && addend->strides[rank - 2] != 0) || (Lk > 1 && addend->strides[rank - 1] != 1))
            return sg_fail(ctx, SG_ERR_SHAPE, "sg_attention addend: one value per key (query stride 0, key stride 1)");
        p.add = (const float *)addend->base + addend->offset;
        p.a_sb1 = rank >= 3 ? addend->strides[rank - 3] : 0;
        p.a_sb0 = rank >= 4 ? addend->strides[rank - 4] : 0;
    }
    if (rank == 3) {  // the single batch axis is b1
        p.q_sb0 = p.k_sb0 = p.v_sb0 = p.o_sb0 = p.a_sb0 = 0;
    }
    p.Lq = (int)Lq; p.Lk = (int)Lk; p.nb1 = (int)nb1;
    p.scale = scale;
    if (nb0 * nb1 > 65535) return sg_fail(ctx, SG_ERR_SHAPE, "sg_attention: more than 65535 (batch x head) pairs");
    // Few workgroups of 128 queries (less than two per compute unit): halving the work units (see the kernel)
    // balances the SIMDs.  The split kernel is held to 168 registers so that three of its workgroups share a
    // compute unit.  Measured at b32 x 12 heads (queries x keys): 23.0 against 25.0 us at 128 x 128 (22.3 with the XCD placement), 37 against
    // 43 at 128 x 256, 63.5 against 76 at 128 x 512, 15 against 22 at 64 x 128; slower once the chip is full anyway.
    const int64_t wgs128 = nb0 * nb1 * ((Lq + 127) / 128);
    bool split = wgs128 < 2 * (int64_t)(ctx->num_cus > 0 ? ctx->num_cus : 256);
    if (ctx->force_attention_split >= 0) split = ctx->force_attention_split != 0;  // measurement switch, fixed at context creation
    const int qb = split ? 64 : 128;
    dim3 grid((unsigned)((Lq + qb - 1) / qb), (unsigned)(nb0 * nb1));
    p.xcd_remap = grid.x > 1 && (grid.x * grid.y) % 8 == 0;
    p.d_gx = sg_make_fastdiv(grid.x);
    p.d_nb1 = sg_make_fastdiv((uint32_t)nb1);
    // the all-aligned instantiation addresses K and V through 32-bit byte offsets from the (batch, head) pair's first row
    const bool fits32 = (Lk + 64) * p.k_sl < (1ll << 29) && (Lk + 64) * p.v_sl < (1ll << 29) && p.k_sl >= 0 && p.v_sl >= 0;
    const bool vec = p.vec_q && p.vec_k && p.vec_v && p.vec_o && fits32;
#define SG_ATTN_LAUNCH(D_, SPLIT_)                                                                                             \
    do {                                                                                                                       \
        if (vec) hipLaunchKernelGGL((attention_kernel<D_, SPLIT_, true>), grid, dim3(64 * NW), 0, ctx->stream, p);            \
        else hipLaunchKernelGGL((attention_kernel<D_, SPLIT_, false>), grid, dim3(64 * NW), 0, ctx->stream, p);               \
    } while (0)
    if (D == 64) {
        if (split) SG_ATTN_LAUNCH(64, true);
        else SG_ATTN_LAUNCH(64, false);
    } else {
        if (split) SG_ATTN_LAUNCH(32, true);
        else SG_ATTN_LAUNCH(32, false);
    }
#undef SG_ATTN_LAUNCH
    SG_CHECK_LAUNCH(ctx, "attention");
    return SG_OK;
}
