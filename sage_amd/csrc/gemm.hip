// fp32 GEMM on the CDNA4 matrix cores (v_mfma_f32_32x32x2_f32), LDS-tiled, for gfx950.
//
// Replaces the reference's GEMM path: Gemm::compute_direct / GemmBatched::compute_direct
// (gemm.rs:176-250, 338-421) launching the vendored XgemmDirect kernels at 8x8 tiles with one
// output per work-item (matmul_direct.opencl:514-709), plus the organize() copies the reference
// needs in front of it (gemm.rs:111-112, 258-259) and the separate bias / activation / residual map
// launches behind it (layers.rs:243-247).
//
// Design:
//   * One workgroup = 4 wavefronts computes a BM x BN tile of C; a wavefront owns a
//     (BM/WAVES_M) x (BN/WAVES_N) sub-tile as TM x TN accumulators of 32x32 (16 VGPRs each).
//   * K is walked in slabs of 16 through a double-buffered LDS: while slab kt is multiplied out of
//     one buffer, slab kt+1 (fetched one iteration earlier into registers) is written to the other
//     and slab kt+2 is being fetched from global memory; one barrier per slab.
//   * Global loads and LDS stores are 16 bytes wide for every layout.  An operand that is
//     contiguous along k (row-major A, transposed B) is kept in LDS as [row][k] and one MFMA operand
//     fetch is a 16-byte read of 4 consecutive k; an operand contiguous along its rows is kept as
//     [k][row] and fetched 4 bytes at a time.  Both orders are bank-conflict free, so all four
//     transpose modes and arbitrarily strided batches run the same loop without any pre-copy or
//     transposition.  (The k index a lane multiplies at step s of a group of four steps is
//     8g + 4*(lane/32) + s for both operands, which is all the MFMA needs.)
//   * Tiles that lie fully inside aligned matrices run an instantiation with no bounds checks at
//     all, whose operand requests are buffer loads (tile descriptor + fixed per-lane offset + scalar
//     slab offset); only edge shapes pay for guarded, zero-filling loads.
//   * On this hardware the vector ALU and the matrix pipe of a SIMD exclude each other, across
//     wavefronts: while one wavefront issues MFMAs back to back no other wavefront of that SIMD
//     gets a vector instruction through (LDS, memory and scalar instructions do issue), and every
//     vector instruction costs the matrix pipe its cycles (about 17 per instruction that interrupts a
//     run of MFMAs).  Hence no vector address arithmetic in the K loop -- global requests are buffer
//     loads with fixed per-lane offsets, LDS reads take fixed per-lane origins plus immediates (nine
//     address additions per two slabs, which the compiler had placed there for paired LDS reads, cost
//     6 % of a 128x96 loop: 1640 cycles per slab against the 1536 of its 24 MFMAs, now 1539) -- a GELU
//     epilogue that reads the normal distribution function from a table in LDS (nine vector
//     instructions per value), and workgroups that walk tiles (the loops of the workgroups on a
//     compute unit run one after the other anyway).
//   * Workgroup ids are remapped so that the ids one XCD receives (id mod 8) cover a compact block
//     of tiles, which keeps the A/B panels a tile group shares inside that XCD's L2.
//   * The epilogue applies alpha, bias[n], activation and a residual on the way out: accumulator
//     blocks go through a per-wavefront LDS stage and leave as 16-byte row segments, in a rolled
//     loop that keeps the kernel's code small.  Unguarded launches without activation or scaling
//     skip all of that: their accumulators start at bias + residual and leave through buffer stores
//     alone, so nothing after the last MFMA costs the matrix pipe a cycle.
//   * Products with at most 16 columns and a few hundred rows (classifier heads) do not use tiles
//     at all: gemm_skinny_kernel gives every output row a wavefront.
// Accumulation order differs from the reference's sequential k (MFMA sums pairs of k, slabs in
// order); the difference is fp32 rounding only and is covered by the 1e-3 GEMM tolerance.
#include "common.h"

#include <atomic>
#include <cmath>
#include <type_traits>

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));  // native vector: stays in registers

constexpr int BK = 16;   // k-slab
constexpr int KPAD = 4;  // row padding of [row][k] LDS tiles (floats)
constexpr int NTHREADS = 256;
constexpr int NUM_XCD = 8;

// Split-K workspace of sg_gemm_noalloc: partial products [split][batch][M][N].  One copy per GPU,
// held until the process ends.  In host code the name `scratch` is only a handle for
// hipGetSymbolAddress; the address kernels and copies use is the per-device pointer below.
constexpr int64_t SCRATCH_FLOATS = (int64_t)SG_GEMM_NOALLOC_SCRATCH_BYTES / 4;
static __device__ __align__(256) float scratch[SCRATCH_FLOATS];
constexpr int MAX_DEVICES = 64;
std::atomic<float *> g_scratch_ptr[MAX_DEVICES];  // device address of `scratch` on each GPU (zero-initialised), set by sg_gemm_device_setup

// The standard normal distribution function on [-6, 6) as 384 cubic pieces (Hermite: exact values and slopes at the
// nodes, worked out in double precision when a device is set up), for the GELU epilogue of the product kernels:
// x * Phi(x) = 0.5 x (1 + erf(x / sqrt 2)).  Piece i covers [-6 + i/32, -6 + (i+1)/32) and holds the coefficients of
// c0 + t (c1 + t (c2 + t c3)), t in [0, 1): the interpolation error is below 2e-9, so what is left is fp32 rounding
// (|error of x Phi(x)| < 5e-7 over [-8, 8], the size of half an ulp of x there).  Nine vector instructions and one
// 16-byte LDS read per value against seventeen for the rational-exponential erf below, and in an epilogue every
// vector instruction is a cycle taken from the matrix pipe.  Below -6 the table's first value is 0 (the product is
// -0, the limit), above 6 its last is 1.
constexpr int GELU_PIECES = 384;
constexpr int GELU_TAB_BYTES = GELU_PIECES * 16;
static __device__ __align__(256) float gelu_tab[GELU_PIECES * 4];
std::atomic<float *> g_gelu_tab_ptr[MAX_DEVICES];  // device address of `gelu_tab` on each GPU, set by sg_gemm_device_setup

// Convolution as a GEMM whose A operand is never materialised: row m of A is output pixel
// (n, oh, ow), column k is filter tap and channel (ky, kx, c), and A[m][k] is read from the image
// x[n, oh*sh - ph + ky*dh, ow*sw - pw + kx*dw, c] (zero outside) while the slab is fetched.
struct ConvG {
    int H, W, C, OW, KW, ohw;      // image height, width, channels; output width; kernel width; OH*OW
    int sh, sw, ph, pw, dh, dw;
    sg_fastdiv d_ohw, d_ow, d_c, d_kw;
    int vec;                       // C % 4 == 0 and the image is 16-byte aligned: four channels per load
    int fast;                      // C % 16 == 0, at most 64 taps, the image below 2^31 bytes: a slab of 16 k is 16 channels
                                   // of ONE tap, so unguarded instantiations can fetch A with buffer loads (see the kernel)
    int KH;                        // kernel height
    uint32_t img_bytes;            // size of the whole image tensor (fast path only)
};

struct GemmP {
    const float *A, *B;
    float *C;
    const float *bias, *res;
    int M, N, K;
    int64_t a_sm, a_sk, b_sk, b_sn, c_sm, r_sm;
    int64_t a_sb0, a_sb1, b_sb0, b_sb1, c_sb0, c_sb1, r_sb0, r_sb1;
    int nb1;  // batch index = b0 * nb1 + b1
    int tiles_m, tiles_n;
    float alpha;
    int act, act_post;
    int vec_a, vec_b;  // 16-byte loads are legal for this operand
    int vec_c, vec_r, vec_bias;  // 16-byte accesses are legal for C rows / residual rows / the bias
    int direct;       // epilogue without vector-ALU work is legal (set by the host, see the kernel): no activation, alpha = 1,
                      // every C / residual offset inside a tile below 2^31 bytes, unguarded instantiation
    const float *gelu;  // the table above when an activation of this launch is GELU (the kernel then has GELU_TAB_BYTES of dynamic LDS), else null
    int k_chunk;      // split-K: workgroup z multiplies k in [z*k_chunk, min(K, (z+1)*k_chunk)); 0 = all of K
    int64_t c_sz;     // split-K: element stride between the partial results of consecutive z
    ConvG conv;       // used by the CONV instantiations only (A is then the image)
};

// erf by the five-term rational-exponential form (Abramowitz & Stegun 7.1.26):
//   erf(x) = 1 - (a1 t + .. + a5 t^5) exp(-x^2),  t = 1 / (1 + p x),  x >= 0,  odd in x,
// with the hardware reciprocal and 2^x.  Absolute error below 6e-7 in fp32 (1.5e-7 from the formula, the
// rest from forming 1 - small in fp32): three orders of magnitude inside the tolerance of a GEMM-bearing
// result.  A dozen instructions, no branch, against about forty with two divergent paths for the
// library routine.  Used where no table is at hand: the split-K second pass and the one-row-per-wavefront kernel
// (the tiled kernels read the table above; the map kernels keep the exact routine).
__device__ __forceinline__ float erf_short(float x) {
    const float ax = __builtin_fabsf(x);
    const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(0.3275911f, ax, 1.0f));
    float q = __builtin_fmaf(1.061405429f, t, -1.453152027f);
    q = __builtin_fmaf(q, t, 1.421413741f);
    q = __builtin_fmaf(q, t, -0.284496736f);
    q = __builtin_fmaf(q, t, 0.254829592f);
    q *= t;
    const float e = __builtin_amdgcn_exp2f(ax * ax * -1.44269504088896340736f);
    return __builtin_copysignf(__builtin_fmaf(-q, e, 1.0f), x);
}

__device__ __forceinline__ float apply_act(float v, int act) {
    if (act == SG_ACT_RELU) return v > 0.0f ? v : 0.0f * v;  // (float)(v>0) * v, nn.rs:39
    if (act == SG_ACT_GELU_ERF) return (v * 0.5f) * (erf_short(v * 0.70710678118654752440f) + 1.0f);
    return v;
}
// GELU through the table (in LDS, 16 bytes per piece)
__device__ __forceinline__ float gelu_lookup(float x, const float *tab) {
    const float u = __builtin_amdgcn_fmed3f(__builtin_fmaf(x, 32.0f, 192.0f), 0.0f, 383.99997f);
    const float t = __builtin_amdgcn_fractf(u);
    const f32x4 c = *reinterpret_cast<const f32x4 *>(reinterpret_cast<const char *>(tab) + ((uint32_t)(int)u << 4));
    return x * __builtin_fmaf(__builtin_fmaf(__builtin_fmaf(c.w, t, c.z), t, c.y), t, c.x);
}
// the same for the four values of a lane, with one uniform branch on the kind instead of four
__device__ __forceinline__ void apply_act4(f32x4 &v, int act, const float *gelu_lds) {
    if (act == SG_ACT_GELU_ERF && gelu_lds) {
        v.x = gelu_lookup(v.x, gelu_lds); v.y = gelu_lookup(v.y, gelu_lds); v.z = gelu_lookup(v.z, gelu_lds); v.w = gelu_lookup(v.w, gelu_lds);
        return;
    }
    if (act == SG_ACT_RELU) {
        v.x = apply_act(v.x, SG_ACT_RELU); v.y = apply_act(v.y, SG_ACT_RELU); v.z = apply_act(v.z, SG_ACT_RELU); v.w = apply_act(v.w, SG_ACT_RELU);
    } else if (act == SG_ACT_GELU_ERF) {
        v.x = apply_act(v.x, SG_ACT_GELU_ERF); v.y = apply_act(v.y, SG_ACT_GELU_ERF); v.z = apply_act(v.z, SG_ACT_GELU_ERF); v.w = apply_act(v.w, SG_ACT_GELU_ERF);
    }
}

// One operand tile (ROWS x BK; rows are m or n indices) on its way from global memory to LDS.
// K_CONTIG: the operand is contiguous along k in global memory.  The tile is then kept in LDS as
// [row][k] (row stride BK+KPAD floats) and an MFMA operand fetch is ONE 16-byte read of 4
// consecutive k; with the padding, 8 consecutive rows cover all 32 banks.  Otherwise the operand is
// contiguous along its rows, the tile is kept as [k][row] (row stride ROWS rounded up to 64 floats, see
// fetch()) and a fetch is a 4-byte read of 32 consecutive floats per half-wave.  Either way global loads
// and LDS stores are 16 bytes wide and no transposition happens on the way.
template <int ROWS, bool K_CONTIG> struct Tile {
    static constexpr int TOTAL = ROWS * BK / 4;                      // float4 per slab
    static constexpr int NV = (TOTAL + NTHREADS - 1) / NTHREADS;     // float4 per thread (last may be partial)
    static constexpr int LD = K_CONTIG ? BK + KPAD : (ROWS + 63) / 64 * 64;
    static constexpr int SIZE = K_CONTIG ? ROWS * LD : BK * LD;      // floats

    // When the slab does not divide evenly over the threads, the surplus slots of the last round
    // repeat earlier ones (same element, same value, same LDS address) instead of branching.
    __device__ static __forceinline__ int slot(int f) { return (TOTAL % NTHREADS == 0 || f < TOTAL) ? f : f - (NV * NTHREADS - TOTAL); }

    // element (row, k) of the slab handled by slot f of this thread
    __device__ static __forceinline__ void where(int f, int &row, int &k) {
        if (K_CONTIG) {
            row = f / (BK / 4);
            k = (f % (BK / 4)) * 4;
        } else {
            k = f / (ROWS / 4);
            row = (f % (ROWS / 4)) * 4;
        }
    }
    __device__ static __forceinline__ int lds_at(int row, int k) { return K_CONTIG ? row * LD + k : k * LD + row; }

    // Unguarded loads (whole tile inside the matrix, 16-byte aligned) are buffer loads: the descriptor holds
    // the tile's base address, the instruction takes a per-lane 32-bit byte offset that is fixed for the
    // kernel (lane_offset(), computed once per item before the loop) and a scalar byte offset for the
    // slab (slab_offset(), one scalar multiply per slab).  The K loop spends no vector instruction and
    // no 64-bit arithmetic on addresses.
    __device__ static __forceinline__ uint32_t lane_offset(int i, uint32_t s_row, uint32_t s_k, int tid) {
        const int f = slot(tid + i * NTHREADS);
        int row, k;
        where(f, row, k);
        return (K_CONTIG ? (uint32_t)row * s_row + (uint32_t)k : (uint32_t)k * s_k + (uint32_t)row) * 4u;
    }
    __device__ static __forceinline__ const float *tile_base(const float *base, int row0, int64_t s_row) {
        return K_CONTIG ? base + (int64_t)row0 * s_row : base + row0;
    }
    __device__ static __forceinline__ __amdgpu_buffer_rsrc_t descriptor(const float *tile) {
        // raw buffer, stride 0, no range limit (the host checked that every offset stays below 2^31), 32-bit data format
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(tile), 0, -1, 0x00020000);
    }
    __device__ static __forceinline__ uint32_t slab_offset(int k0, uint32_t s_k) { return (uint32_t)k0 * (K_CONTIG ? 4u : s_k * 4u); }
    __device__ static __forceinline__ void load_one_fast(f32x4 &r, __amdgpu_buffer_rsrc_t tile, uint32_t lane_off, uint32_t slab_off) {
        typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
        r = __builtin_bit_cast(f32x4, (u32x4)__builtin_amdgcn_raw_buffer_load_b128(tile, lane_off, slab_off, 0));
    }

    // guarded: zero-fill outside [row_lim) x [k_lim), scalar loads when 16-byte loads are not legal
    __device__ static __forceinline__ void load_one_guarded(f32x4 &r, int i, const float *base, int row0, int k0, int row_lim, int k_lim, int64_t s_row,
                                                            int64_t s_k, int vec_ok, int tid) {
        const int f = slot(tid + i * NTHREADS);
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        int row, k;
        where(f, row, k);
        const int gr = row0 + row, gk = k0 + k;
        if (K_CONTIG) {
            if (gr < row_lim) {
                const float *p = base + (int64_t)gr * s_row + gk;
                if (vec_ok && gk + 3 < k_lim) {
                    v = *reinterpret_cast<const f32x4 *>(p);
                } else {
                    if (gk + 0 < k_lim) v.x = p[0];
                    if (gk + 1 < k_lim) v.y = p[1];
                    if (gk + 2 < k_lim) v.z = p[2];
                    if (gk + 3 < k_lim) v.w = p[3];
                }
            }
        } else {
            if (gk < k_lim) {
                const float *p = base + (int64_t)gk * s_k + gr;
                if (vec_ok && gr + 3 < row_lim) {
                    v = *reinterpret_cast<const f32x4 *>(p);
                } else {
                    if (gr + 0 < row_lim) v.x = p[0];
                    if (gr + 1 < row_lim) v.y = p[1];
                    if (gr + 2 < row_lim) v.z = p[2];
                    if (gr + 3 < row_lim) v.w = p[3];
                }
            }
        }
        r = v;
    }

    __device__ static __forceinline__ void store_one(const f32x4 &r, int i, float *lds, int tid) {
        const int f = slot(tid + i * NTHREADS);
        int row, k;
        where(f, row, k);
        *reinterpret_cast<f32x4 *>(&lds[lds_at(row, k)]) = r;
    }

    // MFMA operands of one group of 4 k-steps for one 32-row block: step s of group g multiplies
    // k = 8g + 4*(lane/32) + s.  `at` is the byte offset in LDS of the lane's (row, k = 4*(lane/32)) element of the block
    // in buffer 0 (fetch_origin(), worked out once per kernel); what a fetch adds to it is a compile-time constant, so
    // the loop holds no address arithmetic.  Kept [k][row], a lane's four k are LD floats apart: LD is a multiple of 64
    // floats, which lets two of them share one instruction (a pair of reads 64-dword units apart) from the same address.
    __device__ static __forceinline__ uint32_t fetch_origin(int col, int khalf) { return (uint32_t)(K_CONTIG ? col * LD + 4 * khalf : 4 * khalf * LD + col) * 4u; }
    __device__ static __forceinline__ void fetch(const float *lds, uint32_t at, int buf, int g, float out[4]) {
        const char *p = reinterpret_cast<const char *>(lds) + at + (uint32_t)(buf * SIZE * 4);
        if (K_CONTIG) {
            const f32x4 v = *reinterpret_cast<const f32x4 *>(p + 8 * g * 4);
            out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
        } else {
#pragma unroll
            for (int s = 0; s < 4; ++s) out[s] = *reinterpret_cast<const float *>(p + (8 * g + s) * LD * 4);
        }
    }
};

__device__ __forceinline__ uint32_t fdiv(uint32_t n, sg_fastdiv d) { return (__umulhi(n, d.magic) + n) >> d.shift; }

template <int BM, int BN, int WAVES_M, bool A_KC, bool B_NC, bool GUARD, bool CONV = false, bool DIRECT = false>
__global__ void __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(3, 8))) gemm_mfma_kernel(const GemmP p) {
    static_assert(!CONV || A_KC, "the image-addressed A operand is k-contiguous");
    static_assert(!DIRECT || !GUARD, "the direct write-out belongs to the unguarded instantiations");
    constexpr int WAVES_N = 4 / WAVES_M;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    constexpr int TM = WM / 32, TN = WN / 32;
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of the 32x32 MFMA block");
    typedef Tile<BM, A_KC> TA;
    typedef Tile<BN, !B_NC> TB;
    // Operand buffers during the K loop; afterwards the same memory stages the output blocks.
    constexpr int STAGE_LD = 36, STAGE = 32 * STAGE_LD;  // one 32x32 block per wavefront, padded rows
    constexpr int LDS_OPERANDS = 2 * TA::SIZE + 2 * TB::SIZE;
    constexpr int LDS_FLOATS = LDS_OPERANDS > 4 * STAGE ? LDS_OPERANDS : 4 * STAGE;
    __shared__ __attribute__((aligned(16))) float lds_raw[LDS_FLOATS];
    float(*lds_a)[TA::SIZE] = reinterpret_cast<float(*)[TA::SIZE]>(lds_raw);
    // GELU launches carry the table in dynamic LDS behind the buffers above: every wavefront brings its share (64 pieces
    // per request) with loads that write LDS directly, no register in between; they are the first requests of the
    // kernel, so the wait for the first operand slab and the barrier behind it also make the table visible.
    extern __shared__ __attribute__((aligned(16))) float gelu_dyn[];
    const float *gelu_lds = nullptr;
    if (p.gelu) {
        gelu_lds = gelu_dyn;
        const __amdgpu_buffer_rsrc_t tab_d = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.gelu), 0, GELU_TAB_BYTES, 0x00020000);
        const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
        typedef __attribute__((address_space(3))) void *lds_ptr;
#pragma unroll
        for (int r = 0; r < (GELU_PIECES + NTHREADS - 1) / NTHREADS; ++r) {
            const int first = r * NTHREADS + w * 64;  // this wavefront's first piece of round r
            if (first < GELU_PIECES)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(tab_d, (lds_ptr)(gelu_dyn + first * 4), 16, (uint32_t)((first + (threadIdx.x & 63)) * 16), 0, 0, 0);
        }
    }
    float(*lds_b)[TB::SIZE] = reinterpret_cast<float(*)[TB::SIZE]>(lds_raw + 2 * TA::SIZE);

    // ---- which tile: spread consecutive ids over XCDs, then walk tiles in groups of 8 tile-rows
    // A workgroup walks tiles blockIdx.x, blockIdx.x + gridDim.x, ...  (the host launches one workgroup per
    // tile up to three per compute unit, which is what fits; beyond that the same workgroups take further
    // tiles).  On this hardware a wavefront that issues MFMAs back to back keeps every other wavefront
    // of its SIMD from issuing vector ALU instructions at all, priorities notwithstanding: the K loop
    // below does exactly that, so the workgroups sharing a compute unit run their loops one after the
    // other at full rate and their epilogues all finish together at the end.  Were every tile a
    // workgroup of its own, all slots of all compute units would come free at the same moment and the
    // dispatcher would hand the remaining tiles out unevenly (measured: 4096^3 in 1128 us instead of 950).
    const int ntiles = p.tiles_m * p.tiles_n;
#pragma unroll 1
    for (int tile_id = blockIdx.x; tile_id < ntiles; tile_id += gridDim.x) {
    int pid = tile_id;
    {
        const int per = (ntiles + NUM_XCD - 1) / NUM_XCD;
        int tall = ntiles % NUM_XCD;
        if (tall == 0) tall = NUM_XCD;
        const int xcd = pid % NUM_XCD, local = pid / NUM_XCD;
        pid = xcd < tall ? xcd * per + local : tall * per + (xcd - tall) * (per - 1) + local;
    }
    constexpr int GROUP_M = 8;
    const int in_group = GROUP_M * p.tiles_n;
    const int group = pid / in_group;
    const int first_m = group * GROUP_M;
    const int gsize = min(p.tiles_m - first_m, GROUP_M);
    const int tile_m = first_m + (pid % in_group) % gsize;
    const int tile_n = (pid % in_group) / gsize;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    const int bt0 = blockIdx.y / p.nb1, bt1 = blockIdx.y % p.nb1;
    // split-K: this workgroup's share of the k range, addressed from 0 through shifted bases
    const int k_begin = p.k_chunk ? (int)blockIdx.z * p.k_chunk : 0;
    const int Kloc = p.k_chunk ? min(p.K - k_begin, p.k_chunk) : p.K;
    const float *A = p.A + bt0 * p.a_sb0 + bt1 * p.a_sb1 + (CONV ? 0 : (int64_t)k_begin * p.a_sk);
    const float *B = p.B + bt0 * p.b_sb0 + bt1 * p.b_sb1 + (int64_t)k_begin * p.b_sk;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    float *C = p.C + bt0 * p.c_sb0 + bt1 * p.c_sb1 + (int64_t)blockIdx.z * p.c_sz;
    const float *R = p.res ? p.res + bt0 * p.r_sb0 + bt1 * p.r_sb1 : nullptr;

    // Direct epilogue (unguarded launches without activation or scaling): the accumulators START at bias[n] +
    // residual[m][n] (neither costs a vector instruction once memory has answered) and leave, after the K loop, through buffer stores whose per-lane offset is fixed and whose
    // per-register offset is scalar -- no vector-ALU instruction and no LDS between the last MFMA and the last
    // store.  Vector-ALU work takes its cycles from the matrix pipe of the SIMD whichever wavefront issues it, so
    // only a write-out made of memory instructions alone can overlap the K loop of the next workgroup on the
    // compute unit (or of this workgroup's next tile).  Element r of a 32x32 accumulator block is row
    // (r/4)*8 + (lane/32)*4 + r%4, column lane%32: a store instruction writes two full 128-byte row segments.
    constexpr bool direct = DIRECT;  // (an instantiation of its own: a kernel holds one of the two write-outs, not both)
    typedef unsigned int u32;
    // (descriptors are per tile, hence uniform; the wavefront's block inside the tile is part of the per-lane offset)
    const uint32_t c_lane = ((uint32_t)(wm * WM + (lane >> 5) * 4) * (uint32_t)p.c_sm + (uint32_t)(wn * WN + (lane & 31))) * 4u;
    const uint32_t r_lane = ((uint32_t)(wm * WM + (lane >> 5) * 4) * (uint32_t)p.r_sm + (uint32_t)(wn * WN + (lane & 31))) * 4u;
    const __amdgpu_buffer_rsrc_t c_blk = __builtin_amdgcn_make_buffer_rsrc(C + (int64_t)m0 * p.c_sm + n0, 0, -1, 0x00020000);
    uint32_t bias_lane = (lane >> 5) ? 0x80000000u : (uint32_t)(n0 + wn * WN + (lane & 31)) * 4u;
    float bias_one = (lane >> 5) ? 0.0f : 1.0f;
    asm volatile("" : "+v"(bias_lane), "+v"(bias_one));  // (formed here, among the early vector work, not where they are first used)

    // The requests are ordered so that nothing waits for memory twice: further down, the first two operand slabs,
    // then the residual straight into the accumulator registers, then the bias (a handful of values, added by the
    // matrix pipe in front of the loop).
    floatx16 acc[TM][TN];
    float bias_j[TN];

    // Two register sets for the global fetch: slab s travels through set s&1.
    f32x4 ra0[TA::NV], rb0[TB::NV], ra1[TA::NV], rb1[TB::NV];
    constexpr int NWR = TA::NV + TB::NV;  // 16-byte items per thread and slab (global loads = LDS writes)
    constexpr int NRB = TM + TN;          // operand fetches (one per 32-row block) per group of k-steps
    constexpr int NMFMA = 4 * TM * TN;    // MFMAs per group
    const int a_col = wm * WM + (lane & 31), b_col = wn * WN + (lane & 31), khalf = lane >> 5;
    // where this lane's operands of each 32-row block start in LDS (bytes from lds_raw, buffer 0); opaque to the
    // compiler, which would otherwise fold them into fresh address registers inside the loop
    uint32_t a_at[TM], b_at[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        a_at[i] = TA::fetch_origin(a_col + i * 32, khalf);
        asm volatile("" : "+v"(a_at[i]));
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        b_at[j] = (uint32_t)(2 * TA::SIZE * 4) + TB::fetch_origin(b_col + j * 32, khalf);
        asm volatile("" : "+v"(b_at[j]));
    }
    float a0[TM][4], b0[TN][4], a1[TM][4], b1[TN][4];

    // unguarded path: per-lane byte offsets of this thread's items inside a slab, and the tile bases
    uint32_t off_a[TA::NV], off_b[TB::NV];
#pragma unroll
    for (int i = 0; i < TA::NV; ++i) off_a[i] = TA::lane_offset(i, (uint32_t)p.a_sm, (uint32_t)p.a_sk, tid);
#pragma unroll
    for (int i = 0; i < TB::NV; ++i) off_b[i] = TB::lane_offset(i, (uint32_t)p.b_sn, (uint32_t)p.b_sk, tid);
    const __amdgpu_buffer_rsrc_t a_tile = TA::descriptor(TA::tile_base(A, m0, p.a_sm)), b_tile = TB::descriptor(TB::tile_base(B, n0, p.b_sn));

    // CONV: what does not change over the K loop for this thread's items of an A slab: the image of the
    // item's output pixel, the top-left input coordinates of its window, and its column inside a slab
    const float *cv_img[TA::NV];
    int cv_ih0[TA::NV], cv_iw0[TA::NV], cv_k[TA::NV];
    if (CONV) {
#pragma unroll
        for (int i = 0; i < TA::NV; ++i) {
            int row, k;
            TA::where(TA::slot(tid + i * NTHREADS), row, k);
            const uint32_t m = (uint32_t)(m0 + row);
            const uint32_t n_img = fdiv(m, p.conv.d_ohw), r = m - n_img * (uint32_t)p.conv.ohw;
            const uint32_t oh = fdiv(r, p.conv.d_ow), ow = r - oh * (uint32_t)p.conv.OW;
            cv_img[i] = m < (uint32_t)p.M ? p.A + (int64_t)n_img * p.conv.H * p.conv.W * p.conv.C : nullptr;
            cv_ih0[i] = (int)oh * p.conv.sh - p.conv.ph;
            cv_iw0[i] = (int)ow * p.conv.sw - p.conv.pw;
            cv_k[i] = k_begin + k;
        }
    }
    // CONV without guards (every tile inside the matrices, C % 16 == 0): a slab of 16 k is 16 consecutive channels of
    // ONE filter tap, so an item's address is (its output pixel's window origin + its column: fixed for the kernel, a
    // per-lane 32-bit offset) + (the tap's displacement and the slab's first channel: the same for every lane, a scalar
    // offset) -- the shape of the plain unguarded loads, served by the same buffer-load instruction.  What the image's
    // border adds is one bit per item and tap (is this tap of this pixel's window inside the image?), worked out before
    // the loop; an item whose tap is outside asks for an offset beyond the descriptor's range and receives zeros.
    // Offsets count from `ph` rows and `pw` pixels before the image, which keeps every per-lane offset non-negative.
    uint32_t cf_off[TA::NV];
    uint64_t cf_mask[TA::NV];
    __amdgpu_buffer_rsrc_t cf_img = a_tile;
    if (CONV && !GUARD) {
        const uint32_t lead = ((uint32_t)p.conv.ph * p.conv.W + p.conv.pw) * p.conv.C;  // elements in front of the image
        cf_img = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.A) - lead, 0, (int)(p.conv.img_bytes + lead * 4u), 0x00020000);
#pragma unroll
        for (int i = 0; i < TA::NV; ++i) {
            int row, k;
            TA::where(TA::slot(tid + i * NTHREADS), row, k);
            const uint32_t m = (uint32_t)(m0 + row);
            const uint32_t n_img = fdiv(m, p.conv.d_ohw), r = m - n_img * (uint32_t)p.conv.ohw;
            const uint32_t oh = fdiv(r, p.conv.d_ow), ow = r - oh * (uint32_t)p.conv.OW;
            const int ih0 = (int)oh * p.conv.sh - p.conv.ph, iw0 = (int)ow * p.conv.sw - p.conv.pw;
            cf_off[i] = (uint32_t)(((n_img * (uint32_t)p.conv.H + (uint32_t)(ih0 + p.conv.ph)) * (uint32_t)p.conv.W + (uint32_t)(iw0 + p.conv.pw)) * (uint32_t)p.conv.C + (uint32_t)k) * 4u;
            uint64_t mask = 0, bit = 1;
            for (int ky = 0, ih = ih0; ky < p.conv.KH; ++ky, ih += p.conv.dh) {
                const bool row_inside = (unsigned)ih < (unsigned)p.conv.H;
                for (int kx = 0, iw = iw0; kx < p.conv.KW; ++kx, iw += p.conv.dw, bit <<= 1)
                    if (row_inside && (unsigned)iw < (unsigned)p.conv.W) mask |= bit;
            }
            cf_mask[i] = mask;
        }
    }
    auto conv_fast = [&](f32x4 &r, int i, int k0) {
        const uint32_t kb = (uint32_t)(k_begin + k0);  // the same for every lane: scalar arithmetic
        const uint32_t tap = fdiv(kb, p.conv.d_c), c0 = kb - tap * (uint32_t)p.conv.C;
        const uint32_t ky = fdiv(tap, p.conv.d_kw), kx = tap - ky * (uint32_t)p.conv.KW;
        const uint32_t slab_off = ((ky * (uint32_t)p.conv.dh * (uint32_t)p.conv.W + kx * (uint32_t)p.conv.dw) * (uint32_t)p.conv.C + c0) * 4u;
        const uint32_t lane_off = ((cf_mask[i] >> tap) & 1ull) ? cf_off[i] : 0x80000000u;
        TA::load_one_fast(r, cf_img, lane_off, slab_off);
    };
    auto conv_load = [&](f32x4 &r, int i, int k0) {
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        const int gk = cv_k[i] + k0, k_lim = k_begin + Kloc;
        if (cv_img[i] && gk < k_lim) {
            if (p.conv.vec) {  // four consecutive k are four channels of one tap
                const uint32_t t = fdiv((uint32_t)gk, p.conv.d_c), c = (uint32_t)gk - t * (uint32_t)p.conv.C;
                const uint32_t ky = fdiv(t, p.conv.d_kw), kx = t - ky * (uint32_t)p.conv.KW;
                const int ih = cv_ih0[i] + (int)ky * p.conv.dh, iw = cv_iw0[i] + (int)kx * p.conv.dw;
                if ((unsigned)ih < (unsigned)p.conv.H && (unsigned)iw < (unsigned)p.conv.W)
                    v = *reinterpret_cast<const f32x4 *>(cv_img[i] + ((int64_t)ih * p.conv.W + iw) * p.conv.C + c);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (gk + e >= k_lim) break;
                    const uint32_t t = fdiv((uint32_t)(gk + e), p.conv.d_c), c = (uint32_t)(gk + e) - t * (uint32_t)p.conv.C;
                    const uint32_t ky = fdiv(t, p.conv.d_kw), kx = t - ky * (uint32_t)p.conv.KW;
                    const int ih = cv_ih0[i] + (int)ky * p.conv.dh, iw = cv_iw0[i] + (int)kx * p.conv.dw;
                    if ((unsigned)ih < (unsigned)p.conv.H && (unsigned)iw < (unsigned)p.conv.W)
                        v[e] = cv_img[i][((int64_t)ih * p.conv.W + iw) * p.conv.C + c];
                }
            }
        }
        r = v;
    };

    // item e of a slab: global memory -> registers
#define SG_ITEM_LOAD(e, RA, RB, k0)                                                            \
    do {                                                                                       \
        if ((e) < TA::NV) {                                                                    \
            const int ia = (e) < TA::NV ? (e) : 0;                                         \
            if (CONV && GUARD) conv_load(RA[ia], ia, (k0));                                    \
            else if (CONV) conv_fast(RA[ia], ia, (k0));                                        \
            else if (GUARD) TA::load_one_guarded(RA[ia], ia, A, m0, (k0), p.M, Kloc, p.a_sm, p.a_sk, p.vec_a, tid); \
            else TA::load_one_fast(RA[ia], a_tile, off_a[ia], TA::slab_offset((k0), (uint32_t)p.a_sk)); \
        } else {                                                                               \
            const int ib = (e) >= TA::NV ? (e) - TA::NV : 0;                               \
            if (GUARD) TB::load_one_guarded(RB[ib], ib, B, n0, (k0), p.N, Kloc, p.b_sn, p.b_sk, p.vec_b, tid); \
            else TB::load_one_fast(RB[ib], b_tile, off_b[ib], TB::slab_offset((k0), (uint32_t)p.b_sk)); \
        }                                                                                      \
    } while (0)
    // item e of a slab: registers -> LDS buffer BUF
#define SG_ITEM_STORE(e, RA, RB, BUF)                                                          \
    do {                                                                                       \
        if ((e) < TA::NV) {                                                                    \
            const int ia = (e) < TA::NV ? (e) : 0;                                         \
            TA::store_one(RA[ia], ia, lds_a[BUF], tid);                                        \
        } else {                                                                               \
            const int ib = (e) >= TA::NV ? (e) - TA::NV : 0;                               \
            TB::store_one(RB[ib], ib, lds_b[BUF], tid);                                        \
        }                                                                                      \
    } while (0)
    // fetch e of a group: LDS buffer BUF -> MFMA operand registers of group G
#define SG_ITEM_FETCH(e, BUF, G, AR, BR)                                                       \
    do {                                                                                       \
        if ((e) < TM) {                                                                        \
            const int ia = (e) < TM ? (e) : 0;                                             \
            TA::fetch(lds_raw, a_at[ia], BUF, G, AR[ia]);                                      \
        } else {                                                                               \
            const int ib = (e) >= TM ? (e) - TM : 0;                                       \
            TB::fetch(lds_raw, b_at[ib], BUF, G, BR[ib]);                                      \
        }                                                                                      \
    } while (0)
#define SG_MFMA_OP(ACC, A_, B_) ACC = __builtin_amdgcn_mfma_f32_32x32x2f32(A_, B_, ACC, 0, 0, 0)
#define SG_MFMA(t, AR, BR)                                                                     \
    do {                                                                                       \
        const int s_ = (t) / (TM * TN), i_ = ((t) / TN) % TM, j_ = (t) % TN;               \
        SG_MFMA_OP(acc[i_][j_], AR[i_][s_], BR[j_][s_]);                                      \
    } while (0)

    // Software pipeline of one wavefront, per K slab of 16 (two groups g0, g1 of four MFMA k-steps):
    //   S3  MFMAs of g0 (operands were read during the previous iteration); behind the first of
    //       them, in this order: the LDS writes of slab kt+1 (in registers since iteration kt-2)
    //       to the other buffer, the LDS reads of this slab's g1 operands, and the global requests
    //       for slab kt+3 into the registers just freed
    //   --  barrier: every wavefront's writes are now visible
    //   S5  MFMAs of g1; behind the first of them the LDS reads of the NEXT slab's g0 operands
    // The instruction order is pinned (scheduling barriers between the steps): memory instructions
    // issue in the shadow of a running MFMA, the LDS queue drains during the item-free tail of each
    // group, and the waits in front of the barrier and in front of the next group find it empty.
    // Every LDS read has a whole MFMA group to land, a global fetch has two iterations, and there
    // is one barrier per slab.
    // Hazards: the writes overwrite the buffer last read in the previous iteration; a wavefront can
    // only get there after the previous barrier, which all wavefronts reach after those reads have
    // returned (lgkmcnt(0) precedes the barrier).  The g1 reads see what the previous iteration
    // wrote before that same barrier; the g0 reads see what this iteration wrote before its barrier.
    static_assert(BK == 16, "the pipeline below is written for two groups of four k-steps per slab");
    constexpr int ITEMS3 = 2 * NWR + NRB;
    // Which MFMA of S3 an item is issued behind: LDS writes one per MFMA from the first, then LDS reads
    // two per MFMA, then global requests two per MFMA; the remaining MFMAs of the group run with the
    // LDS queue draining.  (Measured in cycles per slab of a 128x96 tile against other groupings: two
    // LDS writes per MFMA +118, one global request per MFMA +24, all four requests behind one MFMA -10.)
    constexpr int W_PER = 1, R_PER = 2, G_PER = 2;
    constexpr int SW = (NWR + W_PER - 1) / W_PER, SR = (NRB + R_PER - 1) / R_PER;
    // (items that find no slot of their own go behind the last MFMA of the group)
    auto slot3 = [](int e) constexpr { const int t = e < NWR ? e / W_PER : e < NWR + NRB ? SW + (e - NWR) / R_PER : SW + SR + (e - NWR - NRB) / G_PER; return t < NMFMA ? t : NMFMA - 1; };
    constexpr int IPS5 = (NRB + NMFMA - 2) / (NMFMA - 1);
    // The body is unconditional: past the end of K the write goes to a buffer nobody reads again
    // and the fetch re-reads the last slab (unguarded path) or returns zeros (guarded path).  The
    // slab count is rounded up to even; the unguarded path therefore requires K % 32 == 0, the
    // guarded one multiplies a slab of zeros.
    const int nk = ((Kloc + BK - 1) / BK + 1) & ~1;
    const int k_last = GUARD ? (nk + 2) * BK : (nk - 1) * BK;
#define SG_SLAB_BODY(KT, RA, RB)                                                               \
    do {                                                                                       \
        const int cur = (KT) & 1;                                                              \
        const int k_next = min(((KT) + 3) * BK, k_last);                                       \
        _Pragma("unroll") for (int t = 0; t < NMFMA; ++t) {                                    \
            SG_MFMA(t, a0, b0);                                                                \
            __builtin_amdgcn_sched_barrier(0);                                                 \
            _Pragma("unroll") for (int e = 0; e < ITEMS3; ++e) {                               \
                if (slot3(e) != t) continue;                                                   \
                if (e < NWR) SG_ITEM_STORE(e, RA, RB, cur ^ 1);                                \
                else if (e < NWR + NRB) SG_ITEM_FETCH(e - NWR, cur, 1, a1, b1);                \
                else SG_ITEM_LOAD(e - NWR - NRB, RA, RB, k_next);                              \
            }                                                                                  \
            __builtin_amdgcn_sched_barrier(0);                                                 \
        }                                                                                      \
        __syncthreads();                                                                       \
        _Pragma("unroll") for (int t = 0; t < NMFMA; ++t) {                                    \
            SG_MFMA(t, a1, b1);                                                                \
            __builtin_amdgcn_sched_barrier(0);                                                 \
            _Pragma("unroll") for (int e = t * IPS5; e < (t + 1) * IPS5; ++e) {                \
                if (e < NRB) SG_ITEM_FETCH(e, cur ^ 1, 0, a0, b0);                             \
            }                                                                                  \
            __builtin_amdgcn_sched_barrier(0);                                                 \
        }                                                                                      \
    } while (0)

#pragma unroll
    for (int e = 0; e < NWR; ++e) SG_ITEM_LOAD(e, ra0, rb0, 0);
#pragma unroll
    for (int e = 0; e < NWR; ++e) SG_ITEM_LOAD(e, ra1, rb1, BK);
    __builtin_amdgcn_sched_barrier(0);  // (the operand requests above leave before the residual's)
    if (direct && R) {
        const __amdgpu_buffer_rsrc_t r_blk = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(R + (int64_t)m0 * p.r_sm + n0), 0, -1, 0x00020000);
        uint32_t r_row = (uint32_t)p.r_sm * 4u;
        asm volatile("" : "+s"(r_row));  // (scalar offsets formed here, one multiply each, not held in registers from further up)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc[i][j][r] = __builtin_bit_cast(float, (u32)__builtin_amdgcn_raw_buffer_load_b32(
                        r_blk, r_lane, (uint32_t)(i * 32 + (r >> 2) * 8 + (r & 3)) * r_row + (uint32_t)(j * 128), 0));
    } else {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    }
    {
        // (lanes of the upper half, which stand for k = 1 of the MFMA below, ask beyond the descriptor's range and receive 0;
        // so does every lane of a launch without a bias or with the staged epilogue, whose descriptor is empty: no branch
        // here, whose outcome would have to travel to the MFMAs below through a vector register)
        const __amdgpu_buffer_rsrc_t bias_d =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.bias ? p.bias : p.A), 0, direct && p.bias ? p.N * 4 : 0, 0x00020000);
#pragma unroll
        for (int j = 0; j < TN; ++j)
            bias_j[j] = __builtin_bit_cast(float, (u32)__builtin_amdgcn_raw_buffer_load_b32(bias_d, bias_lane, (uint32_t)(j * 128), 0));
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int e = 0; e < NWR; ++e) SG_ITEM_STORE(e, ra0, rb0, 0);
#pragma unroll
    for (int e = 0; e < NWR; ++e) SG_ITEM_LOAD(e, ra0, rb0, min(2 * BK, k_last));
    __syncthreads();
#pragma unroll
    for (int e = 0; e < NRB; ++e) SG_ITEM_FETCH(e, 0, 0, a0, b0);
    if (direct) {
        // acc += ones x bias as one MFMA per block (A = 1 for k = 0 and 0 for k = 1, B = bias[n] for k = 0): the bias
        // joins without a vector instruction.  Vector instructions of a workgroup that enters while an older one streams
        // MFMAs get no issue slot; placed behind the first memory wait they would hold this workgroup's loop back until
        // the older loop has ended (measured: 1.7 us of idle matrix pipe at the hand-over).
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bias_one, bias_j[j], acc[i][j], 0, 0, 0);
    }
    for (int kt = 0; kt < nk; kt += 2) {
        SG_SLAB_BODY(kt, ra1, rb1);
        SG_SLAB_BODY(kt + 1, ra0, rb0);
    }
#undef SG_SLAB_BODY
#undef SG_ITEM_LOAD
#undef SG_ITEM_STORE
#undef SG_ITEM_FETCH
#undef SG_MFMA
#undef SG_MFMA_OP

    // ---- epilogue.  Element r of a 32x32 accumulator block sits at row (r/4)*8 + (lane/32)*4 + r%4,
    // column lane%32.  Each wavefront passes its blocks one at a time through a private 32x32 LDS
    // stage and reads them back as rows, so bias / residual / C move 16 bytes per lane in full
    // 128-byte row segments.  Everything after the staging write is ONE rolled loop over the
    // blocks: the kernel stays a few KB of code instead of an unrolled copy of the activation math
    // per accumulator register, which costs microseconds of instruction fetch on every launch.
    // The bias and residual values of a block are requested one block ahead (the first ones before
    // the barrier), so the rolled loop never waits a full memory round trip per row group; inside
    // the loop the four row groups' residuals sit in a small shift register to keep indices static.
    if (direct) {
        // (the row stride is made opaque here so that the scalar offsets below are formed now, one multiply each,
        // instead of being hoisted above the K loop and held in registers through it)
        uint32_t c_row = (uint32_t)p.c_sm * 4u;
        asm volatile("" : "+s"(c_row));
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float v = acc[i][j][r];  // (a copy: bit-casting the vector element in place reads element 0)
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(u32, v), c_blk, c_lane,
                                                          (uint32_t)(i * 32 + (r >> 2) * 8 + (r & 3)) * c_row + (uint32_t)(j * 128), 0);
                }
        __syncthreads();  // every wavefront has read its last operands: the next tile may overwrite the LDS buffers
        continue;
    }
    float *stage = lds_raw + wave * STAGE;
    const int st_w = (khalf * 4) * STAGE_LD + (lane & 31);        // + ((r/4)*8 + r%4) * STAGE_LD
    const int rd_row = lane >> 3, rd_col = (lane & 7) * 4;          // + 8q rows
    auto request = [&](int blk, f32x4(&res)[4], f32x4 &bias) {
        const int mb = m0 + wm * WM + (blk / TN) * 32, n = n0 + wn * WN + (blk % TN) * 32 + rd_col;
        const bool n_in = !GUARD || n + 3 < p.N;
        bias = f32x4{0.f, 0.f, 0.f, 0.f};
        if (p.bias) {
            if (!GUARD || (p.vec_bias && n_in)) bias = *reinterpret_cast<const f32x4 *>(p.bias + n);
            else {
                if (n + 0 < p.N) bias.x = p.bias[n + 0];
                if (n + 1 < p.N) bias.y = p.bias[n + 1];
                if (n + 2 < p.N) bias.z = p.bias[n + 2];
                if (n + 3 < p.N) bias.w = p.bias[n + 3];
            }
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            res[q] = f32x4{0.f, 0.f, 0.f, 0.f};
            const int m = mb + q * 8 + rd_row;
            if (R && (!GUARD || (m < p.M && n < p.N))) {
                const float *rp = R + (int64_t)m * p.r_sm + n;
                if (!GUARD || (p.vec_r && n_in)) res[q] = *reinterpret_cast<const f32x4 *>(rp);
                else {
                    res[q].x = rp[0];
                    if (n + 1 < p.N) res[q].y = rp[1];
                    if (n + 2 < p.N) res[q].z = rp[2];
                    if (n + 3 < p.N) res[q].w = rp[3];
                }
            }
        }
    };
    f32x4 res_c[4], res_n[4], bias_c, bias_n;
    request(0, res_c, bias_c);
    __syncthreads();  // all operand reads are done; the stage aliases the operand buffers
#pragma unroll 1
    for (int blk = 0; blk < TM * TN; ++blk) {
        // the accumulator block is chosen by a uniform branch so that register indices stay static
#pragma unroll
        for (int ij = 0; ij < TM * TN; ++ij) {
            if (blk == ij) {
#pragma unroll
                for (int r = 0; r < 16; ++r) stage[st_w + ((r >> 2) * 8 + (r & 3)) * STAGE_LD] = acc[ij / TN][ij % TN][r];
            }
        }
        if (TM * TN > 1) request(min(blk + 1, TM * TN - 1), res_n, bias_n);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int mb = m0 + wm * WM + (blk / TN) * 32, n = n0 + wn * WN + (blk % TN) * 32 + rd_col;
        const bool n_in = !GUARD || n + 3 < p.N;
        // The row groups of the block: stage -> alpha, bias, activation, residual, activation -> C.  The launches
        // without an activation (most of them) take a copy of the loop that has no activation code at all.
        auto row_groups = [&](auto with_act) {
            constexpr bool ACT = decltype(with_act)::value;
#pragma unroll 1
            for (int q = 0; q < 4; ++q) {
                const int row = q * 8 + rd_row, m = mb + row;
                f32x4 v = *reinterpret_cast<const f32x4 *>(&stage[row * STAGE_LD + rd_col]);
                const f32x4 res = res_c[0];
                res_c[0] = res_c[1]; res_c[1] = res_c[2]; res_c[2] = res_c[3];
                if (GUARD && (m >= p.M || n >= p.N)) continue;
                if (p.alpha != 1.0f) v *= p.alpha;
                if (p.bias) v += bias_c;
                if (ACT) apply_act4(v, p.act, gelu_lds);
                if (R) v += res;
                if (ACT) apply_act4(v, p.act_post, gelu_lds);
                float *cp = C + (int64_t)m * p.c_sm + n;
                if (!GUARD || (p.vec_c && n_in)) *reinterpret_cast<f32x4 *>(cp) = v;
                else {
                    cp[0] = v.x;
                    if (n + 1 < p.N) cp[1] = v.y;
                    if (n + 2 < p.N) cp[2] = v.z;
                    if (n + 3 < p.N) cp[3] = v.w;
                }
            }
        };
        if (p.act == SG_ACT_NONE && p.act_post == SG_ACT_NONE) row_groups(std::false_type{});
        else row_groups(std::true_type{});
        if (TM * TN > 1) {
#pragma unroll
            for (int q = 0; q < 4; ++q) res_c[q] = res_n[q];
            bias_c = bias_n;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();  // the stage is read out: the next tile's operands may overwrite it
    }  // tiles of this workgroup
}

// Split-K second pass: sums the partial products of the k ranges in ascending order (so the result
// does not depend on scheduling) and applies the epilogue.  ws holds [split][batch][M][N] dense.
template <bool VEC>
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const float *__restrict__ ws, int nsplit, int64_t slice, const GemmP p,
                                                            int64_t total) {
    constexpr int W = VEC ? 4 : 1;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int ncol = p.N / W;
    const int n = (int)(idx % ncol) * W;
    const int64_t row = idx / ncol;
    const int m = (int)(row % p.M);
    const int bt = (int)(row / p.M), bt0 = bt / p.nb1, bt1 = bt % p.nb1;
    const float *src = ws + row * p.N + n;
    float v[W];
#pragma unroll
    for (int i = 0; i < W; ++i) v[i] = 0.0f;
    // eight partial products are requested at a time (one memory round trip per eight) and added in ascending z
    for (int z0 = 0; z0 < nsplit; z0 += 8) {
        f32x4 t[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            t[u] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (z0 + u < nsplit) {
                if (VEC) t[u] = *reinterpret_cast<const f32x4 *>(src + (z0 + u) * slice);
                else t[u].x = src[(z0 + u) * slice];
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if (z0 + u < nsplit) {
#pragma unroll
                for (int i = 0; i < W; ++i) v[i] += t[u][i];
            }
        }
    }
    const float *R = p.res ? p.res + bt0 * p.r_sb0 + bt1 * p.r_sb1 + (int64_t)m * p.r_sm + n : nullptr;
    float *C = p.C + bt0 * p.c_sb0 + bt1 * p.c_sb1 + (int64_t)m * p.c_sm + n;
#pragma unroll
    for (int i = 0; i < W; ++i) {
        float x = v[i];
        if (p.alpha != 1.0f) x *= p.alpha;
        if (p.bias) x += p.bias[n + i];
        x = apply_act(x, p.act);
        if (R) x += R[i];
        x = apply_act(x, p.act_post);
        v[i] = x;
    }
    if (VEC && p.vec_c) *reinterpret_cast<f32x4 *>(C) = f32x4{v[0], v[W > 1 ? 1 : 0], v[W > 2 ? 2 : 0], v[W > 3 ? 3 : 0]};
    else {
#pragma unroll
        for (int i = 0; i < W; ++i) C[i] = v[i];
    }
}

// Products with at most 16 output columns (a classifier head: 128 x 512 x 10, 64 x 768 x 2): an MFMA tile would be
// nearly empty and K would have to be split over workgroups and summed by a second launch to occupy more than two
// compute units.  Here one wavefront owns one output row: its lanes walk k in steps of 64 (A[m, k] is one
// coalesced request per step, the N values of B's row k sit side by side), every lane keeps N partial sums, and
// the wavefront adds them up with xor-shuffles at the end.  The order of the additions is fixed (lane l sums
// k = l, l + 64, ...; then a butterfly over the lanes): the same call gives the same bits.
template <int NMAX>
__global__ void __launch_bounds__(256) gemm_skinny_kernel(const GemmP p) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = blockIdx.x * 4 + wave;
    if (m >= p.M) return;
    float acc[NMAX];
#pragma unroll
    for (int n = 0; n < NMAX; ++n) acc[n] = 0.0f;
    const float *a = p.A + (int64_t)m * p.a_sm;
    constexpr int U = NMAX <= 4 ? 8 : 4;  // requests per operand in flight (more would not fit the registers at 16 columns)
    for (int k0 = 0; k0 < p.K; k0 += 64 * U) {
        float av[U], bv[U][NMAX];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = k0 + u * 64 + lane;
            av[u] = k < p.K ? a[(int64_t)k * p.a_sk] : 0.0f;
#pragma unroll
            for (int n = 0; n < NMAX; ++n) bv[u][n] = (k < p.K && n < p.N) ? p.B[(int64_t)k * p.b_sk + (int64_t)n * p.b_sn] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int n = 0; n < NMAX; ++n) acc[n] = __builtin_fmaf(av[u], bv[u][n], acc[n]);
    }
#pragma unroll
    for (int n = 0; n < NMAX; ++n)
#pragma unroll
        for (int s = 32; s >= 1; s >>= 1) acc[n] += __shfl_xor(acc[n], s, 64);
    // lane n finishes column n
    float v = 0.0f;
#pragma unroll
    for (int n = 0; n < NMAX; ++n)
        if (lane == n) v = acc[n];
    if (lane < p.N) {
        if (p.alpha != 1.0f) v *= p.alpha;
        if (p.bias) v += p.bias[lane];
        v = apply_act(v, p.act);
        if (p.res) v += p.res[(int64_t)m * p.r_sm + lane];
        v = apply_act(v, p.act_post);
        p.C[(int64_t)m * p.c_sm + lane] = v;
    }
}

template <int BM, int BN, int WAVES_M, bool GUARD, bool DIRECT>
void launch_variants(sg_ctx *ctx, const GemmP &p, dim3 grid, dim3 block, unsigned dyn, bool conv, bool a_kc, bool b_nc) {
    if (conv) {  // image-addressed A (sg_conv2d): one instantiation per tile shape
        hipLaunchKernelGGL((gemm_mfma_kernel<BM, BN, WAVES_M, true, true, GUARD, true, DIRECT>), grid, block, dyn, ctx->stream, p);
        return;
    }
    if (a_kc && b_nc) hipLaunchKernelGGL((gemm_mfma_kernel<BM, BN, WAVES_M, true, true, GUARD, false, DIRECT>), grid, block, dyn, ctx->stream, p);
    else if (a_kc && !b_nc) hipLaunchKernelGGL((gemm_mfma_kernel<BM, BN, WAVES_M, true, false, GUARD, false, DIRECT>), grid, block, dyn, ctx->stream, p);
    else if (!a_kc && b_nc) hipLaunchKernelGGL((gemm_mfma_kernel<BM, BN, WAVES_M, false, true, GUARD, false, DIRECT>), grid, block, dyn, ctx->stream, p);
    else hipLaunchKernelGGL((gemm_mfma_kernel<BM, BN, WAVES_M, false, false, GUARD, false, DIRECT>), grid, block, dyn, ctx->stream, p);
}

template <int BM, int BN, int WAVES_M, bool GUARD>
void launch_layouts(sg_ctx *ctx, const GemmP &p_in, dim3 grid, bool a_kc, bool b_nc) {
    GemmP p = p_in;
    const bool gelu = p.act == SG_ACT_GELU_ERF || p.act_post == SG_ACT_GELU_ERF;
    p.gelu = gelu && ctx->device >= 0 && ctx->device < MAX_DEVICES ? g_gelu_tab_ptr[ctx->device].load(std::memory_order_acquire) : nullptr;
    dim3 block(NTHREADS);
    const unsigned dyn = p.gelu ? GELU_TAB_BYTES : 0;
    const bool conv = p.conv.ohw != 0;
    const bool direct = !GUARD && p.direct;
    const int inst[8] = {BM, BN, WAVES_M, conv || a_kc, conv || b_nc, GUARD, conv, direct};
    for (int i = 0; i < 8; ++i) ctx->last_gemm[i] = inst[i];
    if constexpr (!GUARD) {
        if (direct) {
            launch_variants<BM, BN, WAVES_M, false, true>(ctx, p, grid, block, dyn, conv, a_kc, b_nc);
            return;
        }
    }
    launch_variants<BM, BN, WAVES_M, GUARD, false>(ctx, p, grid, block, dyn, conv, a_kc, b_nc);
}

// The epilogue made of buffer stores alone (see the kernel): no activation, no scaling, and every offset inside a
// wavefront's block of C / of the residual below 2^31 bytes.  SAGE_GEMM_DIRECT=0 (read when the context is created)
// switches it off for measurements.
void set_direct(const sg_ctx *ctx, GemmP &p, int bm) {
    const int64_t reach_c = (int64_t)bm * p.c_sm * 4, reach_r = p.res ? (int64_t)bm * p.r_sm * 4 : 0;
    p.direct = ctx->gemm_direct && p.act == SG_ACT_NONE && p.act_post == SG_ACT_NONE && p.alpha == 1.0f && p.c_sm >= 0 && p.r_sm >= 0 &&
               reach_c < (1ll << 31) && reach_r < (1ll << 31);
}

// GUARD = false needs every tile to lie fully inside the matrices and 16-byte loads to be legal.
bool needs_guard(const GemmP &p, int bm, int bn, bool a_kc, bool b_nc) {
    // the unguarded loads address a tile through 32-bit byte offsets (per lane inside a slab, scalar per
    // slab): everything a tile reaches over the whole of K must stay below 2^31 bytes from its base
    const int64_t reach_a = a_kc ? (int64_t)bm * p.a_sm + p.K : (int64_t)p.K * p.a_sk + bm;
    const int64_t reach_b = b_nc ? (int64_t)p.K * p.b_sk + bn : (int64_t)bn * p.b_sn + p.K;
    const bool fits32 = reach_a >= 0 && reach_b >= 0 && reach_a < (1ll << 29) && reach_b < (1ll << 29);
    const bool vec_out = p.vec_c && (!p.res || p.vec_r) && (!p.bias || p.vec_bias);
    // image-addressed A: unguarded when the slabs are single taps (conv.fast) and B, C and the tiling allow it
    if (p.conv.ohw) return !p.conv.fast || p.M % bm != 0 || p.N % bn != 0 || p.K % (2 * BK) != 0 || !p.vec_b || !vec_out || reach_b < 0 || reach_b >= (1ll << 29);
    return p.M % bm != 0 || p.N % bn != 0 || p.K % (2 * BK) != 0 || !p.vec_a || !p.vec_b || !vec_out || !fits32;
}

// How many k ranges to split into.  Splitting pays when the output has too few tiles to occupy the
// chip and K is long: each range becomes its own workgroup (grid z) writing a partial product, and a
// second kernel sums them.  Ranges are multiples of 32 so that the unguarded loop stays legal.
int choose_split(const sg_ctx *ctx, int64_t wgs, int K, bool guarded_loop, int *k_chunk) {
    const int64_t cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
    *k_chunk = 0;
    const int force = ctx->force_gemm_split;  // a measurement switch, fixed when the context was created
    int want;
    if (force) want = force;
    else {
        // The matrix pipe of a compute unit is what a workgroup's loop occupies: two workgroups on one unit take
        // twice as long as one, so the ranges are cut so that tiles x ranges fills the units ONCE (measured on
        // 16, 32 and 64 tiles with K = 576..4608: the time has its minimum at tiles x ranges = 256 and jumps by
        // a quarter right above it).
        if (wgs * 2 > cus) return 1;
        want = (int)(cus / wgs);
        if (want > K / 128) want = K / 128;
        if (want > 128) want = 128;
    }
    if (want < 2) return 1;
    int chunk = ((K + want - 1) / want + 31) / 32 * 32;
    const int nsplit = (K + chunk - 1) / chunk;
    if (nsplit < 2) return 1;
    // A tile multiplies 16 of k in about 0.21 us (more with guarded loads); the second pass and its launch cost
    // about 5 us: the split has to take that many slabs off a workgroup's loop.
    if (!force && (K / 16) * (nsplit - 1) / nsplit < (guarded_loop ? 16 : 24)) return 1;
    *k_chunk = chunk;
    return nsplit;
}

// Where the partial products of a split-K product go: a block from the context's allocator (it counts against
// the capacity; when it does not fit the call fails with SG_ERR_OOM like any other allocation, and the caller's
// eviction loop, session.rs:259-325, frees memory and calls again, instead of silently taking a single-pass
// kernel whose rounding differs), or the static per-device array for the entry point that allocates nothing.
int workspace(sg_ctx *ctx, int64_t floats, bool noalloc, void **ws) {
    if (!noalloc) return sg_alloc(ctx, (uint64_t)floats * sizeof(float), ws);
    if (floats > SCRATCH_FLOATS)
        return sg_fail(ctx, SG_ERR_ARG, "sg_gemm_noalloc: this product runs split-K and needs %lld bytes of workspace, "
                       "more than the %lld-byte static scratch (use sg_gemm)", (long long)floats * 4, (long long)SCRATCH_FLOATS * 4);
    *ws = ctx->device >= 0 && ctx->device < MAX_DEVICES ? g_scratch_ptr[ctx->device].load(std::memory_order_acquire) : nullptr;
    if (!*ws) return sg_fail(ctx, SG_ERR_DEVICE, "sg_gemm_noalloc: the static scratch of device %d was not set up", ctx->device);
    return SG_OK;
}

// The first pass of a split-K product: raw partial products [split][batch][M][N] into the workspace, no epilogue.
GemmP partial_pass(const GemmP &p, float *ws, int64_t slice, int k_chunk) {
    GemmP q = p;
    q.C = ws;
    q.c_sm = p.N; q.c_sb1 = (int64_t)p.M * p.N; q.c_sb0 = q.c_sb1 * p.nb1; q.c_sz = slice;
    q.k_chunk = k_chunk;
    q.bias = nullptr; q.res = nullptr; q.alpha = 1.0f; q.act = SG_ACT_NONE; q.act_post = SG_ACT_NONE;
    q.vec_c = p.N % 4 == 0;
    return q;
}

void launch_splitk_reduce(sg_ctx *ctx, const GemmP &p, const float *ws, int nsplit, int64_t slice);

template <int BM, int BN, int WAVES_M>
int launch_cfg(sg_ctx *ctx, GemmP &p, int batch, bool a_kc, bool b_nc, bool noalloc) {
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    int k_chunk = 0;
    const int nsplit = choose_split(ctx, (int64_t)p.tiles_m * p.tiles_n * batch, p.K, needs_guard(p, BM, BN, a_kc, b_nc), &k_chunk);
    if (nsplit > 1) {
        const int64_t slice = (int64_t)batch * p.M * p.N;
        void *ws = nullptr;
        const int rc_ws = workspace(ctx, (int64_t)nsplit * slice, noalloc, &ws);
        if (rc_ws != SG_OK) return rc_ws;
        GemmP q = partial_pass(p, (float *)ws, slice, k_chunk);
        set_direct(ctx, q, BM);
        dim3 grid((unsigned)(p.tiles_m * p.tiles_n), (unsigned)batch, (unsigned)nsplit);
        if (needs_guard(q, BM, BN, a_kc, b_nc)) launch_layouts<BM, BN, WAVES_M, true>(ctx, q, grid, a_kc, b_nc);
        else launch_layouts<BM, BN, WAVES_M, false>(ctx, q, grid, a_kc, b_nc);
        SG_CHECK_LAUNCH(ctx, "gemm (split-K pass 1)");
        launch_splitk_reduce(ctx, p, (const float *)ws, nsplit, slice);
        SG_CHECK_LAUNCH(ctx, "gemm (split-K pass 2)");
        // the static scratch stays; a block from the allocator returns to the context's cache (later users of either
        // are ordered behind these kernels on the stream)
        return noalloc ? SG_OK : sg_free(ctx, ws);
    }
    // one workgroup per tile while they all fit at once (three per compute unit), else that many workgroups
    // walking the tiles; a batched product keeps one workgroup per tile and batch entry
    const int64_t ntiles = (int64_t)p.tiles_m * p.tiles_n, resident = 3 * (int64_t)ctx->num_cus;
    dim3 grid((unsigned)(batch == 1 && ntiles > resident ? resident : ntiles), (unsigned)batch);
    set_direct(ctx, p, BM);
    if (needs_guard(p, BM, BN, a_kc, b_nc)) launch_layouts<BM, BN, WAVES_M, true>(ctx, p, grid, a_kc, b_nc);
    else launch_layouts<BM, BN, WAVES_M, false>(ctx, p, grid, a_kc, b_nc);
    SG_CHECK_LAUNCH(ctx, "gemm");
    return SG_OK;
}

struct TileCfg { int bm, bn, waves_m; };
const TileCfg kTileCfgs[] = {{128, 128, 2}, {128, 96, 4}, {128, 64, 2}, {64, 64, 2}};

int choose_tile(const sg_ctx *ctx, int M, int N, int K, int batch) {
    if (ctx->force_gemm_tile >= 0) return ctx->force_gemm_tile;
    const int64_t cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
    int best = 3;
    double best_score = -1.0;
    for (int c = 0; c < 4; ++c) {
        const int64_t tm = (M + kTileCfgs[c].bm - 1) / kTileCfgs[c].bm, tn = (N + kTileCfgs[c].bn - 1) / kTileCfgs[c].bn;
        const int64_t tiles = tm * tn * batch;
        const int64_t rounds = (tiles + cus - 1) / cus;
        // useful work / (rounds * cus * tile area): fill of the last round and of edge tiles
        const double useful = (double)M * N * batch;
        const double spent = (double)rounds * cus * kTileCfgs[c].bm * kTileCfgs[c].bn;
        double score = useful / spent;
        // larger tiles re-read less of A and B: small bonus.  With a short K a workgroup is mostly its fixed
        // latencies (first operands, write-out), which more, smaller workgroups on a compute unit overlap:
        // the bonus goes the other way (25088 x 49 x 64: 9.4 us in 64x64 tiles against 13.9 in 128x64).
        score *= 1.0 + 0.05 * (K > 256 ? 3 - c : c);
        if (score > best_score) {
            best_score = score;
            best = c;
        }
    }
    return best;
}

void launch_splitk_reduce(sg_ctx *ctx, const GemmP &p, const float *ws, int nsplit, int64_t slice) {
    const bool vec = p.N % 4 == 0;
    const int64_t total = slice / (vec ? 4 : 1);
    dim3 rgrid((unsigned)((total + 255) / 256));
    if (vec) hipLaunchKernelGGL((splitk_reduce_kernel<true>), rgrid, dim3(256), 0, ctx->stream, ws, nsplit, slice, p, total);
    else hipLaunchKernelGGL((splitk_reduce_kernel<false>), rgrid, dim3(256), 0, ctx->stream, ws, nsplit, slice, p, total);
}

int launch_gemm(sg_ctx *ctx, GemmP &p, int batch, bool a_kc, bool b_nc, bool noalloc) {
    // (a wavefront per row pays while the rows are few: 128 x 512 x 10 takes 7.7 us against 13.7 for tile + split-K + second pass,
    // 64 x 768 x 2 4.5 against 13; a lane's reads of B are 4 bytes at a stride of N floats, so thousands of rows are better off
    // in MFMA tiles: 1024 x 512 x 16 took 18 us, 32768 x 768 x 2 43 us)
    if (batch == 1 && p.conv.ohw == 0 && p.N <= 16 && p.M <= 512 && ctx->force_gemm_tile < 0 && ctx->force_gemm_split == 0) {
        dim3 grid((unsigned)((p.M + 3) / 4));
        const int inst[8] = {-1, p.N <= 4 ? 4 : 16, 0, 0, 0, 0, 0, 0};  // sg_gemm_last_kernel_name: gemm_skinny_kernel<NMAX>
        for (int i = 0; i < 8; ++i) ctx->last_gemm[i] = inst[i];
        if (p.N <= 4) hipLaunchKernelGGL((gemm_skinny_kernel<4>), grid, dim3(256), 0, ctx->stream, p);
        else hipLaunchKernelGGL((gemm_skinny_kernel<16>), grid, dim3(256), 0, ctx->stream, p);
        SG_CHECK_LAUNCH(ctx, "gemm (skinny)");
        return SG_OK;
    }
    switch (choose_tile(ctx, p.M, p.N, p.K, batch)) {
    case 0: return launch_cfg<128, 128, 2>(ctx, p, batch, a_kc, b_nc, noalloc);
    case 1: return launch_cfg<128, 96, 4>(ctx, p, batch, a_kc, b_nc, noalloc);
    case 2: return launch_cfg<128, 64, 2>(ctx, p, batch, a_kc, b_nc, noalloc);
    default: return launch_cfg<64, 64, 2>(ctx, p, batch, a_kc, b_nc, noalloc);
    }
}

bool ptr_aligned16(const float *p) { return ((uintptr_t)p) % 16 == 0; }

// a: [b0,b1,M,K] strides (.., sm, sk) ; b: [b0,b1,K,N] ; c: [b0,b1,M,N]
struct Mat {
    const float *ptr;
    int64_t sb0, sb1, s_row, s_col;
};

int run(sg_ctx *ctx, int M, int N, int K, int nb0, int nb1, Mat a, Mat b, Mat c, const sg_gemm_epilogue *epi, bool noalloc = false,
        const ConvG *conv = nullptr) {
    if (M < 1 || N < 1 || K < 1) return sg_fail(ctx, SG_ERR_SHAPE, "gemm: empty dimension");
    // Which axis of each operand is the contiguous one.  An axis of extent 1 may carry any stride.
    bool a_kc, b_nc;
    if (a.s_col == 1) a_kc = true;
    else if (a.s_row == 1) a_kc = false;
    else if (K == 1) { a_kc = true; a.s_col = 1; }
    else if (M == 1) { a_kc = false; a.s_row = 1; }
    else return sg_fail(ctx, SG_ERR_SHAPE, "gemm: A needs a unit stride on one of its two axes");
    if (b.s_col == 1) b_nc = true;
    else if (b.s_row == 1) b_nc = false;
    else if (N == 1) { b_nc = true; b.s_col = 1; }
    else if (K == 1) { b_nc = false; b.s_row = 1; }
    else return sg_fail(ctx, SG_ERR_SHAPE, "gemm: B needs a unit stride on one of its two axes");
    if (c.s_col != 1 && N != 1) return sg_fail(ctx, SG_ERR_SHAPE, "gemm: C needs a unit stride on its last axis");
    GemmP p{};
    p.A = a.ptr; p.B = b.ptr; p.C = (float *)c.ptr;
    p.M = M; p.N = N; p.K = K;
    p.a_sm = a.s_row; p.a_sk = a.s_col; p.b_sk = b.s_row; p.b_sn = b.s_col; p.c_sm = c.s_row;
    p.a_sb0 = a.sb0; p.a_sb1 = a.sb1; p.b_sb0 = b.sb0; p.b_sb1 = b.sb1; p.c_sb0 = c.sb0; p.c_sb1 = c.sb1;
    p.nb1 = nb1;
    if (conv) p.conv = *conv;
    p.alpha = 1.0f; p.act = SG_ACT_NONE; p.act_post = SG_ACT_NONE;
    auto mult4 = [](int64_t v) { return v % 4 == 0; };
    p.vec_a = ptr_aligned16(a.ptr) && mult4(a_kc ? p.a_sm : p.a_sk) && mult4(a.sb0) && mult4(a.sb1);
    p.vec_b = ptr_aligned16(b.ptr) && mult4(b_nc ? p.b_sk : p.b_sn) && mult4(b.sb0) && mult4(b.sb1);
    p.vec_c = c.s_col == 1 && ptr_aligned16(c.ptr) && mult4(p.c_sm) && mult4(c.sb0) && mult4(c.sb1);
    if (epi) {
        p.alpha = epi->alpha;
        p.act = epi->act; p.act_post = epi->act_post;
        if (p.act < 0 || p.act > SG_ACT_GELU_ERF || p.act_post < 0 || p.act_post > SG_ACT_GELU_ERF) return sg_fail(ctx, SG_ERR_ARG, "gemm: unknown activation");
        if (epi->bias) {
            const sg_tensor *t = epi->bias;
            int rc = sg_validate_tensor(ctx, t, "gemm bias");
            if (rc != SG_OK) return rc;
            if (t->dtype != SG_FLOAT) return sg_fail(ctx, SG_ERR_DTYPE, "gemm: bias must be fp32");
            if (sg_numel(t) != N || !sg_is_dense(t)) return sg_fail(ctx, SG_ERR_SHAPE, "gemm: bias must be dense with N = %d elements", N);
            p.bias = (const float *)t->base + t->offset;
            p.vec_bias = ptr_aligned16(p.bias);
        }
        if (epi->residual) {
            const sg_tensor *t = epi->residual;
            int rc = sg_validate_tensor(ctx, t, "gemm residual");
            if (rc != SG_OK) return rc;
            if (t->dtype != SG_FLOAT) return sg_fail(ctx, SG_ERR_DTYPE, "gemm: residual must be fp32");
            // accepted layouts: [M,N] for a single matrix, [batch,M,N] with the batch axes flattened, or [b0,b1,M,N]
            const int r = t->rank;
            if (r < 2 || t->extents[r - 1] != N || t->extents[r - 2] != M || (N != 1 && t->strides[r - 1] != 1))
                return sg_fail(ctx, SG_ERR_SHAPE, "gemm: residual must be [..,M,N] with unit last stride");
            int64_t lead = 1;
            for (int i = 0; i < r - 2; ++i) lead *= t->extents[i];
            if (lead != (int64_t)nb0 * nb1) return sg_fail(ctx, SG_ERR_SHAPE, "gemm: residual batch extents differ from C's");
            p.res = (const float *)t->base + t->offset;
            p.r_sm = t->strides[r - 2];
            p.r_sb1 = r >= 3 ? t->strides[r - 3] : 0;
            p.r_sb0 = r >= 4 ? t->strides[r - 4] : 0;
            if (r == 3) {  // one flattened batch axis: entry b0 * nb1 + b1
                p.r_sb1 = t->strides[0];
                p.r_sb0 = (int64_t)nb1 * t->strides[0];
            }
            if (r > 4) return sg_fail(ctx, SG_ERR_SHAPE, "gemm: residual rank above 4");
            p.vec_r = (N == 1 || t->strides[r - 1] == 1) && ptr_aligned16(p.res) && mult4(p.r_sm) && mult4(p.r_sb0) && mult4(p.r_sb1);
        }
    }
    return launch_gemm(ctx, p, nb0 * nb1, a_kc, b_nc, noalloc);
}

int check_f32(sg_ctx *ctx, const sg_tensor *a, const sg_tensor *b, const sg_tensor *c, const char *who) {
    int rc;
    if ((rc = sg_validate_tensor(ctx, a, who)) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, b, who)) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, c, who)) != SG_OK) return rc;
    if (a->dtype != SG_FLOAT || b->dtype != SG_FLOAT || c->dtype != SG_FLOAT) return sg_fail(ctx, SG_ERR_DTYPE, "%s: fp32 only", who);
    return SG_OK;
}

}  // namespace

extern "C" int sg_gemm_last_kernel_name(sg_ctx *ctx, char *buf, uint64_t cap) {
    if (!ctx || !buf || cap < 8) return SG_ERR_ARG;
    const int *t = ctx->last_gemm;
    if (t[0] == 0) return sg_fail(ctx, SG_ERR_ARG, "sg_gemm_last_kernel_name: no product has been launched on this context");
    if (t[0] < 0) {
        snprintf(buf, cap, "gemm_skinny_kernel<%d>", t[1]);
        return SG_OK;
    }
    snprintf(buf, cap, "gemm_mfma_kernel<%d, %d, %d, %s, %s, %s, %s, %s>", t[0], t[1], t[2], t[3] ? "true" : "false", t[4] ? "true" : "false",
             t[5] ? "true" : "false", t[6] ? "true" : "false", t[7] ? "true" : "false");
    return SG_OK;
}

namespace {
int gemm_rank2(sg_ctx *ctx, int ta, int tb, const sg_tensor *a, const sg_tensor *b, const sg_tensor *c, const sg_gemm_epilogue *epi,
               bool noalloc) {
    if (!ctx) return SG_ERR_ARG;
    int rc = check_f32(ctx, a, b, c, "sg_gemm");
    if (rc != SG_OK) return rc;
    if (a->rank != 2 || b->rank != 2 || c->rank != 2) return sg_fail(ctx, SG_ERR_SHAPE, "sg_gemm: rank-2 tensors expected");
    // (height, chan1, width, chan2) of gemm.rs:118-124
    const int64_t M = a->extents[ta ? 1 : 0], K = a->extents[ta ? 0 : 1];
    const int64_t N = b->extents[tb ? 0 : 1], K2 = b->extents[tb ? 1 : 0];
    if (K != K2) return sg_fail(ctx, SG_ERR_SHAPE, "sg_gemm: inner dimensions %lld and %lld differ (gemm.rs:124)", (long long)K, (long long)K2);
    if (c->extents[0] != M || c->extents[1] != N) return sg_fail(ctx, SG_ERR_SHAPE, "sg_gemm: C must be [%lld,%lld]", (long long)M, (long long)N);
    // ld = strides[0]; the stored inner axis must be contiguous (gemm.rs:111-112 organizes first)
    if ((a->extents[1] != 1 && a->strides[1] != 1) || (b->extents[1] != 1 && b->strides[1] != 1) || (c->extents[1] != 1 && c->strides[1] != 1))
        return sg_fail(ctx, SG_ERR_SHAPE, "sg_gemm: operands must have a unit inner stride (use sg_matmul_strided for general layouts)");
    Mat ma{(const float *)a->base + a->offset, 0, 0, ta ? 1 : a->strides[0], ta ? a->strides[0] : 1};
    Mat mb{(const float *)b->base + b->offset, 0, 0, tb ? 1 : b->strides[0], tb ? b->strides[0] : 1};
    Mat mc{(const float *)c->base + c->offset, 0, 0, c->strides[0], 1};
    return run(ctx, (int)M, (int)N, (int)K, 1, 1, ma, mb, mc, epi, noalloc);
}
}  // namespace

extern "C" int sg_gemm(sg_ctx *ctx, int ta, int tb, const sg_tensor *a, const sg_tensor *b, const sg_tensor *c,
                       const sg_gemm_epilogue *epi) {
    return gemm_rank2(ctx, ta, tb, a, b, c, epi, false);
}

// The same product with the split-K workspace in the static per-device array: no allocation of any kind.
extern "C" int sg_gemm_noalloc(sg_ctx *ctx, int ta, int tb, const sg_tensor *a, const sg_tensor *b, const sg_tensor *c,
                               const sg_gemm_epilogue *epi) {
    return gemm_rank2(ctx, ta, tb, a, b, c, epi, true);
}

// conv_2d (conv.rs:61-96) in one launch: the [N*OH*OW, KH*KW*C] column matrix of im2col is never written;
// the GEMM's A operand is read from the image through the window arithmetic of Im2col (conv.rs:304-349).
extern "C" int sg_conv2d(sg_ctx *ctx, const sg_tensor *x, const sg_tensor *filter, const sg_tensor *out, const int32_t stride[2],
                         const int32_t pad[2], const int32_t dil[2], const sg_gemm_epilogue *epi) {
    if (!ctx || !stride || !pad || !dil) return SG_ERR_ARG;
    int rc = check_f32(ctx, x, filter, out, "sg_conv2d");
    if (rc != SG_OK) return rc;
    if (x->rank != 4 || filter->rank != 4 || out->rank != 4) return sg_fail(ctx, SG_ERR_SHAPE, "sg_conv2d: x [N,H,W,C], filter [KH,KW,C,OC], out [N,OH,OW,OC] (conv.rs:70, 199)");
    if (!sg_is_dense(x) || !sg_is_dense(filter) || !sg_is_dense(out)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_conv2d: operands must be dense (conv.rs:200)");
    for (int i = 0; i < 2; ++i)
        if (stride[i] < 1 || pad[i] < 0 || dil[i] < 0) return sg_fail(ctx, SG_ERR_ARG, "sg_conv2d: bad geometry");
    const int64_t N = x->extents[0], H = x->extents[1], W = x->extents[2], Cc = x->extents[3];
    const int64_t KH = filter->extents[0], KW = filter->extents[1], OC = filter->extents[3];
    if (filter->extents[2] != Cc) return sg_fail(ctx, SG_ERR_SHAPE, "sg_conv2d: filter has %lld input channels, the image %lld (conv.rs:86)", (long long)filter->extents[2], (long long)Cc);
    // conv_size (conv.rs:47-59); every pair is {w, h}
    const int64_t OW = (W + 2 * pad[0] - (int64_t)dil[0] * (KW - 1) - 1) / stride[0] + 1;
    const int64_t OH = (H + 2 * pad[1] - (int64_t)dil[1] * (KH - 1) - 1) / stride[1] + 1;
    if (OW < 1 || OH < 1) return sg_fail(ctx, SG_ERR_SHAPE, "sg_conv2d: kernel larger than padded image");
    const int64_t want[4] = {N, OH, OW, OC};
    for (int a = 0; a < 4; ++a)
        if (out->extents[a] != want[a]) return sg_fail(ctx, SG_ERR_SHAPE, "sg_conv2d: out extent[%d] = %lld, expected %lld", a, (long long)out->extents[a], (long long)want[a]);
    // Taps that lie in the padding for EVERY output pixel multiply zeros (a 3x3 window with padding 1 over a 1x1 image has
    // one tap inside the image, over a 2-pixel-high image with stride 2 two of its three rows).  When the taps some
    // pixel can reach form a block of the filter that is contiguous in memory (one row of taps, or whole rows), the
    // product runs over that block alone: a smaller kernel window with the padding reduced accordingly.  The terms
    // left out are exact zeros, so the sum keeps its value; K, and with it the split over workgroups, shrinks.
    int64_t ky0 = 0, ky1 = KH - 1, kx0 = 0, kx1 = KW - 1;
    int64_t ph = pad[1], pw = pad[0];
    {
        auto reach = [](int64_t k, int64_t n_out, int64_t s, int64_t p, int64_t d, int64_t extent) {  // some output pixel reads the image through tap k
            for (int64_t o = 0; o < n_out; ++o) {
                const int64_t i = o * s - p + k * d;
                if (i >= 0 && i < extent) return true;
                if (i >= extent) break;
            }
            return false;
        };
        int64_t a = 0, b = KH - 1, c = 0, e = KW - 1;
        while (a < b && !reach(a, OH, stride[1], pad[1], dil[1], H)) ++a;
        while (b > a && !reach(b, OH, stride[1], pad[1], dil[1], H)) --b;
        while (c < e && !reach(c, OW, stride[0], pad[0], dil[0], W)) ++c;
        while (e > c && !reach(e, OW, stride[0], pad[0], dil[0], W)) --e;
        const bool smaller = a > 0 || b < KH - 1 || c > 0 || e < KW - 1;
        const bool contiguous = a == b || (c == 0 && e == KW - 1);
        if (smaller && contiguous && pad[1] - a * dil[1] >= 0 && pad[0] - c * dil[0] >= 0 && dil[0] > 0 && dil[1] > 0) {
            ky0 = a; ky1 = b; kx0 = c; kx1 = e;
            ph = pad[1] - a * dil[1];
            pw = pad[0] - c * dil[0];
        }
    }
    const int64_t KHe = ky1 - ky0 + 1, KWe = kx1 - kx0 + 1;  // the window the product walks
    const int64_t M = N * OH * OW, K = KHe * KWe * Cc;
    if (M >= (1ll << 31) || K >= (1ll << 31)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_conv2d: more than 2^31-1 output pixels or filter taps");
    ConvG g{};
    g.H = (int)H; g.W = (int)W; g.C = (int)Cc; g.OW = (int)OW; g.KW = (int)KWe; g.ohw = (int)(OH * OW);
    g.sw = stride[0]; g.sh = stride[1]; g.pw = (int)pw; g.ph = (int)ph; g.dw = dil[0]; g.dh = dil[1];
    g.d_ohw = sg_make_fastdiv((uint32_t)g.ohw); g.d_ow = sg_make_fastdiv((uint32_t)OW);
    g.d_c = sg_make_fastdiv((uint32_t)Cc); g.d_kw = sg_make_fastdiv((uint32_t)KWe);
    const float *img = (const float *)x->base + x->offset;
    g.vec = Cc % 4 == 0 && ptr_aligned16(img);
    g.KH = (int)KHe;
    const int64_t img_bytes = N * H * W * Cc * 4, lead_bytes = (ph * W + pw) * Cc * 4;
    // The unguarded loads send an outside tap to lane offset 2^31 and rely on the descriptor's range check, which
    // compares against (range - scalar offset): that difference must not wrap, so the largest scalar offset of
    // the loop (last tap's displacement + the last 16-channel slab, + the 64 bytes it reads) has to lie inside
    // the range; a dilation or padding larger than the image (N = 1) can exceed it and takes the guarded loads.
    const int64_t max_slab_off = (((KHe - 1) * (int64_t)dil[1] * W + (KWe - 1) * (int64_t)dil[0]) * Cc + (Cc >= 16 ? Cc - 16 : 0)) * 4 + 64;
    g.fast = Cc % 16 == 0 && ptr_aligned16(img) && KHe * KWe <= 64 && img_bytes + lead_bytes < (1ll << 31) &&
             max_slab_off <= img_bytes + lead_bytes;
    g.img_bytes = g.fast ? (uint32_t)img_bytes : 0u;
    // A = the virtual [M, K] column matrix (row stride K, never dereferenced through it), B = filter as [K, OC], C = out as [M, OC]
    Mat ma{img, 0, 0, K, 1};
    // B = the filter rows of the taps walked: [ky0..ky1] x [kx0..kx1] x C, contiguous by the test above
    Mat mb{(const float *)filter->base + filter->offset + (ky0 * KW + kx0) * Cc * OC, 0, 0, OC, 1};
    Mat mc{(const float *)out->base + out->offset, 0, 0, OC, 1};
    return run(ctx, (int)M, (int)OC, (int)K, 1, 1, ma, mb, mc, epi, false, &g);
}

// Called by sg_ctx_create with the context's device current: resolves the device address of `scratch`
// on that GPU once (each GPU holds its own copy of the array at its own address).
int sg_gemm_device_setup(sg_ctx *ctx) {
    if (ctx->device < 0 || ctx->device >= MAX_DEVICES) return SG_OK;  // sg_gemm_noalloc reports it when used
    if (g_scratch_ptr[ctx->device].load(std::memory_order_acquire) && g_gelu_tab_ptr[ctx->device].load(std::memory_order_acquire)) return SG_OK;
    if (!g_gelu_tab_ptr[ctx->device].load(std::memory_order_acquire)) {
        static float host_tab[GELU_PIECES * 4];  // (the same values whichever thread writes them)
        const double h = 1.0 / 32.0;
        auto Phi = [](double x) { return 0.5 * erfc(-x * 0.70710678118654752440); };
        auto phi = [](double x) { return exp(-0.5 * x * x) * 0.39894228040143267794; };
        for (int i = 0; i < GELU_PIECES; ++i) {
            const double x0 = -6.0 + i * h, x1 = x0 + h;
            const double v0 = i == 0 ? 0.0 : Phi(x0), v1 = Phi(x1), s0 = phi(x0) * h, s1 = phi(x1) * h, d = v1 - v0;
            host_tab[4 * i + 0] = (float)v0;
            host_tab[4 * i + 1] = (float)s0;
            host_tab[4 * i + 2] = (float)(3.0 * d - 2.0 * s0 - s1);
            host_tab[4 * i + 3] = (float)(s0 + s1 - 2.0 * d);
        }
        SG_HIP(ctx, hipMemcpyToSymbol(HIP_SYMBOL(gelu_tab), host_tab, sizeof host_tab));
        float *tab = nullptr;
        SG_HIP(ctx, hipGetSymbolAddress((void **)&tab, HIP_SYMBOL(gelu_tab)));
        g_gelu_tab_ptr[ctx->device].store(tab, std::memory_order_release);
    }
    float *ptr = nullptr;
    SG_HIP(ctx, hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
    // contexts created at the same time on several threads all resolve the same address: whichever store lands is right
    g_scratch_ptr[ctx->device].store(ptr, std::memory_order_release);
    return SG_OK;
}

extern "C" int sg_gemm_batched(sg_ctx *ctx, int ta, int tb, const sg_tensor *a, const sg_tensor *b, const sg_tensor *c,
                               const sg_gemm_epilogue *epi) {
    if (!ctx) return SG_ERR_ARG;
    int rc = check_f32(ctx, a, b, c, "sg_gemm_batched");
    if (rc != SG_OK) return rc;
    if (a->rank != 3 || b->rank != 3 || c->rank != 3) return sg_fail(ctx, SG_ERR_SHAPE, "sg_gemm_batched: rank-3 tensors expected");
    const int64_t batch = a->extents[0];
    const int64_t M = a->extents[ta ? 2 : 1], K = a->extents[ta ? 1 : 2];
    const int64_t N = b->extents[tb ? 1 : 2], K2 = b->extents[tb ? 2 : 1];
    if (b->extents[0] != batch || c->extents[0] != batch) return sg_fail(ctx, SG_ERR_SHAPE, "sg_gemm_batched: batch extents differ (gemm.rs:261)");
    if (K != K2) return sg_fail(ctx, SG_ERR_SHAPE, "sg_gemm_batched: inner dimensions differ (gemm.rs:276)");
    if (c->extents[1] != M || c->extents[2] != N) return sg_fail(ctx, SG_ERR_SHAPE, "sg_gemm_batched: C must be [%lld,%lld,%lld]", (long long)batch, (long long)M, (long long)N);
    if ((a->extents[2] != 1 && a->strides[2] != 1) || (b->extents[2] != 1 && b->strides[2] != 1) || (c->extents[2] != 1 && c->strides[2] != 1))
        return sg_fail(ctx, SG_ERR_SHAPE, "sg_gemm_batched: operands must have a unit inner stride");
    Mat ma{(const float *)a->base + a->offset, a->strides[0], 0, ta ? 1 : a->strides[1], ta ? a->strides[1] : 1};
    Mat mb{(const float *)b->base + b->offset, b->strides[0], 0, tb ? 1 : b->strides[1], tb ? b->strides[1] : 1};
    Mat mc{(const float *)c->base + c->offset, c->strides[0], 0, c->strides[1], 1};
    return run(ctx, (int)M, (int)N, (int)K, (int)batch, 1, ma, mb, mc, epi);
}

extern "C" int sg_matmul_strided(sg_ctx *ctx, const sg_tensor *a, const sg_tensor *b, const sg_tensor *c, const sg_gemm_epilogue *epi) {
    if (!ctx) return SG_ERR_ARG;
    int rc = check_f32(ctx, a, b, c, "sg_matmul_strided");
    if (rc != SG_OK) return rc;
    const int r = a->rank;
    if (r < 2 || r > 4 || b->rank != r || c->rank != r) return sg_fail(ctx, SG_ERR_SHAPE, "sg_matmul_strided: ranks must agree and be 2..4");
    const int64_t M = a->extents[r - 2], K = a->extents[r - 1], N = b->extents[r - 1];
    if (b->extents[r - 2] != K) return sg_fail(ctx, SG_ERR_SHAPE, "sg_matmul_strided: inner dimensions differ");
    if (c->extents[r - 2] != M || c->extents[r - 1] != N) return sg_fail(ctx, SG_ERR_SHAPE, "sg_matmul_strided: C extents do not match");
    int64_t nb[2] = {1, 1};
    int64_t sa[2] = {0, 0}, sb[2] = {0, 0}, sc[2] = {0, 0};
    for (int i = 0; i < r - 2; ++i) {
        const int slot = 2 - (r - 2) + i;
        if (b->extents[i] != a->extents[i] || c->extents[i] != a->extents[i]) return sg_fail(ctx, SG_ERR_SHAPE, "sg_matmul_strided: batch extents differ");
        nb[slot] = a->extents[i];
        sa[slot] = a->strides[i];
        sb[slot] = b->strides[i];
        sc[slot] = c->strides[i];
    }
    Mat ma{(const float *)a->base + a->offset, sa[0], sa[1], a->strides[r - 2], a->strides[r - 1]};
    Mat mb{(const float *)b->base + b->offset, sb[0], sb[1], b->strides[r - 2], b->strides[r - 1]};
    Mat mc{(const float *)c->base + c->offset, sc[0], sc[1], c->strides[r - 2], c->strides[r - 1]};
    return run(ctx, (int)M, (int)N, (int)K, (int)nb[0], (int)nb[1], ma, mb, mc, epi);
}
