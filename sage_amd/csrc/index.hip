// Indexing kernels for gfx950: gather, scatter, unslice, concat, im2col, col2im, pooling, fill.
//
// These replace the reference's generated kernels of ops/core.rs (gather core.rs:674-705, scatter
// :784-819, unslice :591-600, concat :917-924) and ops/conv.rs (im2col conv.rs:304-349, col2im
// conv.rs:418-473).  They are data movement (col2im and pooling add): results are bit-exact.  Each thread
// owns consecutive output elements along the innermost (contiguous) output axis so stores are coalesced.
// Coordinates come from a mixed-radix decomposition of the thread's linear index, where the reference
// divides and takes remainders per axis and element (core.rs:162-167): here the index space is collapsed
// on the host first (axes of extent 1 vanish, neighbouring axes that every operand walks like one axis
// merge) and what remains is decomposed with multiply-high magic numbers, so no kernel divides in
// hardware; im2col is parallel over every output element instead of looping batch*KH*KW inside a work-item.
#include "common.h"

namespace {

// Index space of a kernel after the host has collapsed it: extents with their multiply-high magic numbers (no
// hardware division on the device; the outermost axis needs none) and up to three stride sets over them.
struct Dims {
    int n;
    uint32_t ext[SG_MAX_RANK];
    sg_fastdiv div[SG_MAX_RANK];
    uint32_t stride[3][SG_MAX_RANK];
};

__device__ __forceinline__ uint32_t fdiv(uint32_t n, sg_fastdiv d) { return (__umulhi(n, d.magic) + n) >> d.shift; }

// Collapses the index space `ext` walked by n_sets stride sets: axes of extent 1 vanish and two neighbouring axes
// merge when every stride set steps through them like through one axis (stride[a] == ext[a+1] * stride[a+1]).
// `keep` (or -1) names an axis that must stay on its own (the gather / scatter axis, whose coordinate is replaced
// by an index); *keep_out receives its position after the collapse.  A dense tensor becomes one axis, a row gather two.
Dims collapse(int rank, const int64_t *ext, int n_sets, const int64_t *const *strides, int keep, int *keep_out) {
    int64_t e[SG_MAX_RANK], st[3][SG_MAX_RANK];
    bool is_keep[SG_MAX_RANK];
    int n = 0;
    for (int a = 0; a < rank; ++a) {
        if (ext[a] == 1 && a != keep) continue;
        const bool merge = n > 0 && a != keep && !is_keep[n - 1] && [&] {
            for (int k = 0; k < n_sets; ++k)
                if (st[k][n - 1] != ext[a] * strides[k][a]) return false;
            return true;
        }();
        if (merge) {
            e[n - 1] *= ext[a];
            for (int k = 0; k < n_sets; ++k) st[k][n - 1] = strides[k][a];
        } else {
            e[n] = ext[a];
            for (int k = 0; k < n_sets; ++k) st[k][n] = strides[k][a];
            is_keep[n] = a == keep;
            ++n;
        }
    }
    if (n == 0) {  // a single element
        e[0] = 1;
        for (int k = 0; k < n_sets; ++k) st[k][0] = 0;
        is_keep[0] = false;
        n = 1;
    }
    Dims d{};
    d.n = n;
    if (keep_out) *keep_out = -1;
    for (int i = 0; i < SG_MAX_RANK; ++i) {
        d.ext[i] = i < n ? (uint32_t)e[i] : 1u;
        d.div[i] = sg_make_fastdiv(d.ext[i]);
        for (int k = 0; k < 3; ++k) d.stride[k][i] = i < n && k < n_sets ? (uint32_t)st[k][i] : 0u;
        if (i < n && is_keep[i] && keep_out) *keep_out = i;
    }
    return d;
}

__global__ void __launch_bounds__(256) fill_u32_kernel(uint32_t *__restrict__ p, uint32_t v, uint64_t n) {
    uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    const uint64_t step = (uint64_t)gridDim.x * 256u;
    for (; i < n; i += step) p[i] = v;
}

// out[gid] = x[x_off + sum_i (i == axis ? ind[...] : c_i) * xstride_i]; c from ind's extents (collapsed on the host).
// Stride set 0 walks ind, set 1 walks x.
__global__ void __launch_bounds__(256) gather_kernel(const uint32_t *__restrict__ x, const uint32_t *__restrict__ ind,
                                                     uint32_t *__restrict__ y, uint32_t n, Dims d, int axis,
                                                     uint32_t x_off, uint32_t ind_off) {
    uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= n) return;
    uint32_t rem = gid, ioff = ind_off, xo = x_off;
    for (int a = d.n - 1; a >= 0; --a) {
        const uint32_t q = a ? fdiv(rem, d.div[a]) : 0u;
        const uint32_t c = rem - q * d.ext[a];
        rem = q;
        ioff += c * d.stride[0][a];
        if (a != axis) xo += c * d.stride[1][a];
    }
    const uint32_t target = ind[ioff];
    y[gid] = x[xo + target * d.stride[1][axis]];
}

// Row gather: x [V, E] with unit inner stride, one index per output row (the index tensor is expanded along the
// inner axis with stride 0, as Embedding::pass builds it, layers.rs:430-446): a thread copies 16 bytes of a row.
// The general kernel above moves 4 bytes per thread behind a division per axis.
__global__ void __launch_bounds__(256) gather_rows_kernel(const uint32_t *__restrict__ x, const uint32_t *__restrict__ ind,
                                                          uint32_t *__restrict__ y, uint32_t n_vec, uint32_t vec_per_row, sg_fastdiv d_row,
                                                          uint32_t x_row_stride, uint32_t ind_row_stride, uint32_t x_off, uint32_t ind_off) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= n_vec) return;
    const uint32_t row = fdiv(gid, d_row), c = gid - row * vec_per_row;
    const uint32_t target = ind[ind_off + row * ind_row_stride];
    *reinterpret_cast<u32x4 *>(y + (size_t)gid * 4u) = *reinterpret_cast<const u32x4 *>(x + x_off + (size_t)target * x_row_stride + c * 4u);
}

template <class T>
__global__ void __launch_bounds__(256) scatter_add_kernel(const T *__restrict__ x, const uint32_t *__restrict__ ind, T *__restrict__ y,
                                                          uint32_t n, Dims d, int axis, uint32_t x_off, uint32_t ind_off) {
    // stride set 0 walks ind, 1 walks x, 2 walks y
    uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= n) return;
    uint32_t rem = gid, ioff = ind_off, xo = x_off, yo = 0;
    for (int a = d.n - 1; a >= 0; --a) {
        const uint32_t q = a ? fdiv(rem, d.div[a]) : 0u;
        const uint32_t c = rem - q * d.ext[a];
        rem = q;
        ioff += c * d.stride[0][a];
        xo += c * d.stride[1][a];
        if (a != axis) yo += c * d.stride[2][a];
    }
    yo += ind[ioff] * d.stride[2][axis];
    atomicAdd(&y[yo], x[xo]);
}

// strided window copy: y[ydims(c)] = x[xdims(c)], c enumerates x's extents
__global__ void __launch_bounds__(256) window_copy_kernel(const uint32_t *__restrict__ x, uint32_t *__restrict__ y, uint32_t n,
                                                          Dims d, uint32_t x_off, uint32_t y_off) {
    // stride set 0 walks x, 1 walks y
    uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= n) return;
    uint32_t rem = gid, xo = x_off, yo = y_off;
    for (int a = d.n - 1; a >= 0; --a) {
        const uint32_t q = a ? fdiv(rem, d.div[a]) : 0u;
        const uint32_t c = rem - q * d.ext[a];
        rem = q;
        xo += c * d.stride[0][a];
        yo += c * d.stride[1][a];
    }
    y[yo] = x[xo];
}

struct Im2colP {
    int batch, chan, img_w, img_h, col_w, col_h, ker_w, ker_h, stride_w, stride_h, pad_w, pad_h, dil_w, dil_h;
    // magic numbers for the decompositions below, set by finish(): channel groups per pixel, column / image / kernel
    // extents, and the strides (col2im divides by them)
    sg_fastdiv d_cv, d_col_w, d_col_h, d_ker_w, d_ker_h, d_img_w, d_img_h, d_stride_w, d_stride_h;
    void finish(int vec) {
        d_cv = sg_make_fastdiv((uint32_t)(chan / vec));
        d_col_w = sg_make_fastdiv((uint32_t)col_w); d_col_h = sg_make_fastdiv((uint32_t)col_h);
        d_ker_w = sg_make_fastdiv((uint32_t)ker_w); d_ker_h = sg_make_fastdiv((uint32_t)ker_h);
        d_img_w = sg_make_fastdiv((uint32_t)img_w); d_img_h = sg_make_fastdiv((uint32_t)img_h);
        d_stride_w = sg_make_fastdiv((uint32_t)stride_w); d_stride_h = sg_make_fastdiv((uint32_t)stride_h);
    }
};

// rem -> (rem / d, rem % d) by multiply-high
__device__ __forceinline__ uint32_t split(uint32_t &rem, uint32_t d, sg_fastdiv m) {
    const uint32_t q = fdiv(rem, m), r = rem - q * d;
    rem = q;
    return r;
}

// Pooling without the column tensor: out[n, oy, ox, c] = reduce over (ky, kx) of the window the reference's
// max_pool_2d / avg_pool_2d first copy out with im2col and then reduce over axes [3, 4] (conv.rs:143-165).
// Pixels outside the image count as zeros, as they do in the column tensor; the accumulator starts at 0
// (ref_zero, reduce.rs:282) or at the operator's identity; the window is walked in the order of the
// reference's reduce kernel (first reduced axis, ky, innermost).  One thread per VEC channels of one output pixel.
template <int VEC>
__global__ void __launch_bounds__(256) pool2d_kernel(const float *__restrict__ img, float *__restrict__ out, uint32_t n_vec, Im2colP p,
                                                     int op, int ref_zero) {
    uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= n_vec) return;
    uint32_t rem = gid;
    const uint32_t c = split(rem, (uint32_t)p.chan / VEC, p.d_cv) * VEC;
    const uint32_t ox = split(rem, (uint32_t)p.col_w, p.d_col_w);
    const uint32_t oy = split(rem, (uint32_t)p.col_h, p.d_col_h);
    const uint32_t n = rem;
    const float start = ref_zero ? 0.0f : (op == SG_R_SUM ? 0.0f : op == SG_R_PROD ? 1.0f : op == SG_R_MAX ? -__builtin_inff() : __builtin_inff());
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = start;
    const float *base = img + (size_t)n * p.img_h * p.img_w * p.chan + c;
    // up to four taps of a window column are requested before the first of them is combined (in tap order, so
    // the result is that of the plain loop, which would wait for each tap in turn)
    for (int kx = 0; kx < p.ker_w; ++kx) {
        const int ix = (int)ox * p.stride_w - p.pad_w + kx * p.dil_w;
        const bool col_inside = ix >= 0 && ix < p.img_w;
        for (int ky0 = 0; ky0 < p.ker_h; ky0 += 4) {
            float v[4][VEC];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int iy = (int)oy * p.stride_h - p.pad_h + (ky0 + u) * p.dil_h;
#pragma unroll
                for (int e = 0; e < VEC; ++e) v[u][e] = 0.0f;
                if (ky0 + u < p.ker_h && col_inside && iy >= 0 && iy < p.img_h) {
                    const float *q = base + ((size_t)iy * p.img_w + ix) * p.chan;
                    if (VEC == 4) {
                        const float4 t = *reinterpret_cast<const float4 *>(q);
                        v[u][0] = t.x; v[u][1 % VEC] = t.y; v[u][2 % VEC] = t.z; v[u][3 % VEC] = t.w;
                    } else {
                        v[u][0] = q[0];
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (ky0 + u >= p.ker_h) break;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float a = acc[e], b = v[u][e];
                    acc[e] = op == SG_R_SUM ? a + b : op == SG_R_PROD ? a * b : op == SG_R_MAX ? (a < b ? b : a) : (b < a ? b : a);
                }
            }
        }
    }
    float *dst = out + (size_t)gid * VEC;
    if (VEC == 4) *reinterpret_cast<float4 *>(dst) = make_float4(acc[0], acc[1 % VEC], acc[2 % VEC], acc[3 % VEC]);
    else dst[0] = acc[0];
}

// One thread per VEC consecutive channels of one (n, oy, ox, ky, kx) cell of the column tensor.
template <int VEC>
__global__ void __launch_bounds__(256) im2col_kernel(const float *__restrict__ img, float *__restrict__ col, uint32_t n_vec, Im2colP p) {
    uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= n_vec) return;
    uint32_t rem = gid;
    const uint32_t c = split(rem, (uint32_t)p.chan / VEC, p.d_cv) * VEC;
    const uint32_t kx = split(rem, (uint32_t)p.ker_w, p.d_ker_w);
    const uint32_t ky = split(rem, (uint32_t)p.ker_h, p.d_ker_h);
    const uint32_t ox = split(rem, (uint32_t)p.col_w, p.d_col_w);
    const uint32_t oy = split(rem, (uint32_t)p.col_h, p.d_col_h);
    const uint32_t n = rem;
    const int ix = (int)ox * p.stride_w - p.pad_w + (int)kx * p.dil_w;
    const int iy = (int)oy * p.stride_h - p.pad_h + (int)ky * p.dil_h;
    const bool inside = ix >= 0 && ix < p.img_w && iy >= 0 && iy < p.img_h;
    const size_t src = (((size_t)n * p.img_h + (inside ? iy : 0)) * p.img_w + (inside ? ix : 0)) * p.chan + c;
    if (VEC == 4) {
        float4 v = inside ? *reinterpret_cast<const float4 *>(img + src) : make_float4(0.f, 0.f, 0.f, 0.f);
        *reinterpret_cast<float4 *>(col + (size_t)gid * 4) = v;
    } else {
        col[gid] = inside ? img[src] : 0.0f;
    }
}

// Col2im::compute (conv.rs:405-500), the adjoint of im2col: out[n, y, x, c] is the sum of every column entry that
// im2col copied from that pixel.  Tap-centric: tap (ky, kx) of output cell (oy, ox) was read from pixel
// (oy*stride_h - pad_h + ky*dil_h, ox*stride_w - pad_w + kx*dil_w), so for each tap the one cell that read THIS pixel
// through it is found by solving for (oy, ox): the remainder of (y + pad_h - ky*dil_h) by stride_h must vanish and
// the quotient must be a row of the column tensor, likewise across.  One thread per VEC channels of a pixel; the
// divisions by the strides are multiply-highs, nothing in the loop divides.
// Order of the float additions: the reference's work-item walks the cells with ox ascending outside and oy
// ascending inside; a larger ox means a smaller kx, so the taps run kx descending outside, ky descending inside and
// the sum is bit-identical to the reference's.  Where the two dilations differ the reference's kernel takes its
// tap indices from the wrong dilation (conv.rs:463-465) and reads entries of other taps or past its buffer: it
// defines no result there; this kernel returns the adjoint.
template <int VEC>
__global__ void __launch_bounds__(256) col2im_kernel(const float *__restrict__ col, float *__restrict__ img, uint32_t n_out, Im2colP p) {
    typedef float vec_t __attribute__((ext_vector_type(VEC)));
    const uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= n_out) return;
    uint32_t rem = gid;
    const uint32_t c = split(rem, (uint32_t)p.chan / VEC, p.d_cv) * VEC;
    const uint32_t x = split(rem, (uint32_t)p.img_w, p.d_img_w);
    const uint32_t y = split(rem, (uint32_t)p.img_h, p.d_img_h);
    const uint32_t n = rem;
    const float *cb = col + (size_t)n * p.col_h * p.col_w * p.ker_h * p.ker_w * p.chan + c;
    vec_t val = 0.0f;
    for (int kx = p.ker_w - 1; kx >= 0; --kx) {
        const int ax = (int)x + p.pad_w - kx * p.dil_w;  // = ox * stride_w for the cell that read this pixel through kx
        if (ax < 0) continue;
        const uint32_t ox = fdiv((uint32_t)ax, p.d_stride_w);
        if (ox * (uint32_t)p.stride_w != (uint32_t)ax || ox >= (uint32_t)p.col_w) continue;
        for (int ky = p.ker_h - 1; ky >= 0; --ky) {
            const int ay = (int)y + p.pad_h - ky * p.dil_h;
            if (ay < 0) continue;
            const uint32_t oy = fdiv((uint32_t)ay, p.d_stride_h);
            if (oy * (uint32_t)p.stride_h != (uint32_t)ay || oy >= (uint32_t)p.col_h) continue;
            val += *reinterpret_cast<const vec_t *>(cb + (size_t)(((oy * p.col_w + ox) * p.ker_h + ky) * p.ker_w + kx) * p.chan);
        }
    }
    *reinterpret_cast<vec_t *>(img + (size_t)gid * VEC) = val;
}

}  // namespace

extern "C" int sg_fill_u32(sg_ctx *ctx, void *dst_dev, uint32_t pattern, uint64_t count) {
    if (!ctx || (!dst_dev && count)) return SG_ERR_ARG;
    if (!count) return SG_OK;
    uint64_t blocks = (count + 255) / 256;
    if (blocks > 65535ull * 16) blocks = 65535ull * 16;
    hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (uint32_t *)dst_dev, pattern, count);
    SG_CHECK_LAUNCH(ctx, "fill");
    return SG_OK;
}

extern "C" int sg_gather(sg_ctx *ctx, int axis, const sg_tensor *x, const sg_tensor *ind, const sg_tensor *out) {
    if (!ctx) return SG_ERR_ARG;
    int rc;
    if ((rc = sg_validate_tensor(ctx, x, "sg_gather x")) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, ind, "sg_gather ind")) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, out, "sg_gather out")) != SG_OK) return rc;
    if (x->rank != ind->rank) return sg_fail(ctx, SG_ERR_SHAPE, "sg_gather: x and ind ranks differ (core.rs:631)");
    if (axis < 0 || axis >= x->rank) return sg_fail(ctx, SG_ERR_SHAPE, "sg_gather: axis out of range");
    if (ind->dtype != SG_UINT && ind->dtype != SG_INT) return sg_fail(ctx, SG_ERR_DTYPE, "sg_gather: ind must be uint or int");
    if (out->dtype != x->dtype) return sg_fail(ctx, SG_ERR_DTYPE, "sg_gather: out dtype differs from x");
    if (!sg_is_dense(out) || sg_numel(out) != sg_numel(ind)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_gather: out must be dense with ind's extents (core.rs:640)");
    for (int a = 0; a < x->rank; ++a)
        if (a != axis && ind->extents[a] > x->extents[a])
            return sg_fail(ctx, SG_ERR_SHAPE, "sg_gather: ind extent[%d] exceeds x's", a);
    const uint32_t n = (uint32_t)sg_numel(ind);
    if (n == 0) return SG_OK;
    if (x->rank == 2 && axis == 0 && ind->extents[1] > 1 && ind->strides[1] == 0 && x->strides[1] == 1 && ind->extents[1] % 4 == 0 &&
        x->strides[0] % 4 == 0 && x->offset % 4 == 0 && (uintptr_t)x->base % 16 == 0 && ((uintptr_t)out->base + (uint64_t)out->offset * 4) % 16 == 0 &&
        x->strides[0] >= 0 && ind->strides[0] >= 0 && x->strides[0] < (1ll << 31) && ind->strides[0] < (1ll << 31)) {
        const uint32_t vec_per_row = (uint32_t)(ind->extents[1] / 4), n_vec = n / 4;
        hipLaunchKernelGGL(gather_rows_kernel, dim3((n_vec + 255) / 256), dim3(256), 0, ctx->stream, (const uint32_t *)x->base,
                           (const uint32_t *)ind->base, (uint32_t *)out->base + out->offset, n_vec, vec_per_row, sg_make_fastdiv(vec_per_row),
                           (uint32_t)x->strides[0], (uint32_t)ind->strides[0], (uint32_t)x->offset, (uint32_t)ind->offset);
        SG_CHECK_LAUNCH(ctx, "gather (rows)");
        return SG_OK;
    }
    int axis_c = 0;
    const int64_t *sets[2] = {ind->strides, x->strides};
    const Dims d = collapse(ind->rank, ind->extents, 2, sets, axis, &axis_c);
    hipLaunchKernelGGL(gather_kernel, dim3((n + 255) / 256), dim3(256), 0, ctx->stream, (const uint32_t *)x->base, (const uint32_t *)ind->base,
                       (uint32_t *)out->base + out->offset, n, d, axis_c, (uint32_t)x->offset, (uint32_t)ind->offset);
    SG_CHECK_LAUNCH(ctx, "gather");
    return SG_OK;
}

extern "C" int sg_scatter(sg_ctx *ctx, int axis, const sg_tensor *x, const sg_tensor *ind, const sg_tensor *out) {
    if (!ctx) return SG_ERR_ARG;
    int rc;
    if ((rc = sg_validate_tensor(ctx, x, "sg_scatter x")) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, ind, "sg_scatter ind")) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, out, "sg_scatter out")) != SG_OK) return rc;
    if (x->rank != ind->rank || out->rank != x->rank) return sg_fail(ctx, SG_ERR_SHAPE, "sg_scatter: ranks differ (core.rs:736-737)");
    if (axis < 0 || axis >= x->rank) return sg_fail(ctx, SG_ERR_SHAPE, "sg_scatter: axis out of range");
    if (ind->dtype != SG_UINT && ind->dtype != SG_INT) return sg_fail(ctx, SG_ERR_DTYPE, "sg_scatter: ind must be uint or int");
    if (out->dtype != x->dtype) return sg_fail(ctx, SG_ERR_DTYPE, "sg_scatter: out dtype differs from x");
    if (!sg_is_dense(out)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_scatter: out must be dense row-major");
    int64_t ds[SG_MAX_RANK];
    sg_default_strides(ind->extents, ind->rank, ds);
    for (int a = 0; a < ind->rank; ++a) {
        if (ind->extents[a] != 1 && ind->strides[a] != ds[a])
            return sg_fail(ctx, SG_ERR_SHAPE, "sg_scatter: ind must have default strides (the reference decomposes by ind's own strides, core.rs:770)");
        if (ind->extents[a] > x->extents[a]) return sg_fail(ctx, SG_ERR_SHAPE, "sg_scatter: ind extent[%d] exceeds x's", a);
        if (a != axis && ind->extents[a] > out->extents[a]) return sg_fail(ctx, SG_ERR_SHAPE, "sg_scatter: ind extent[%d] exceeds out's", a);
    }
    if ((rc = sg_fill_u32(ctx, (uint32_t *)out->base + out->offset, 0u, (uint64_t)sg_numel(out))) != SG_OK) return rc;
    const uint32_t n = (uint32_t)sg_numel(ind);
    int axis_c = 0;
    const int64_t *sets[3] = {ind->strides, x->strides, out->strides};
    const Dims d = collapse(ind->rank, ind->extents, 3, sets, axis, &axis_c);
    dim3 grid((n + 255) / 256);
    if (x->dtype == SG_FLOAT)
        hipLaunchKernelGGL((scatter_add_kernel<float>), grid, dim3(256), 0, ctx->stream, (const float *)x->base, (const uint32_t *)ind->base,
                           (float *)out->base + out->offset, n, d, axis_c, (uint32_t)x->offset, (uint32_t)ind->offset);
    else
        hipLaunchKernelGGL((scatter_add_kernel<unsigned>), grid, dim3(256), 0, ctx->stream, (const unsigned *)x->base, (const uint32_t *)ind->base,
                           (unsigned *)out->base + out->offset, n, d, axis_c, (uint32_t)x->offset, (uint32_t)ind->offset);
    SG_CHECK_LAUNCH(ctx, "scatter");
    return SG_OK;
}

extern "C" int sg_unslice(sg_ctx *ctx, int axis, int64_t start, const sg_tensor *x, const sg_tensor *out) {
    if (!ctx) return SG_ERR_ARG;
    int rc;
    if ((rc = sg_validate_tensor(ctx, x, "sg_unslice x")) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, out, "sg_unslice out")) != SG_OK) return rc;
    if (x->rank != out->rank || axis < 0 || axis >= x->rank) return sg_fail(ctx, SG_ERR_SHAPE, "sg_unslice: rank/axis mismatch");
    if (x->dtype != out->dtype) return sg_fail(ctx, SG_ERR_DTYPE, "sg_unslice: dtype mismatch");
    if (!sg_is_dense(out)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_unslice: out must be dense row-major");
    for (int a = 0; a < x->rank; ++a) {
        if (a == axis ? (start < 0 || start + x->extents[a] > out->extents[a]) : x->extents[a] != out->extents[a])
            return sg_fail(ctx, SG_ERR_SHAPE, "sg_unslice: window does not fit (core.rs:534)");
    }
    if ((rc = sg_fill_u32(ctx, (uint32_t *)out->base + out->offset, 0u, (uint64_t)sg_numel(out))) != SG_OK) return rc;
    const uint32_t n = (uint32_t)sg_numel(x);
    const int64_t *sets[2] = {x->strides, out->strides};
    const Dims d = collapse(x->rank, x->extents, 2, sets, -1, nullptr);
    hipLaunchKernelGGL(window_copy_kernel, dim3((n + 255) / 256), dim3(256), 0, ctx->stream, (const uint32_t *)x->base, (uint32_t *)out->base, n,
                       d, (uint32_t)x->offset, (uint32_t)(out->offset + start * out->strides[axis]));
    SG_CHECK_LAUNCH(ctx, "unslice");
    return SG_OK;
}

extern "C" int sg_concat(sg_ctx *ctx, int axis, const sg_tensor *in, int n_in, const sg_tensor *out) {
    if (!ctx) return SG_ERR_ARG;
    if (!in || n_in < 1) return sg_fail(ctx, SG_ERR_ARG, "sg_concat: no inputs");
    int rc;
    if ((rc = sg_validate_tensor(ctx, out, "sg_concat out")) != SG_OK) return rc;
    if (axis < 0 || axis >= out->rank) return sg_fail(ctx, SG_ERR_SHAPE, "sg_concat: axis out of range");
    if (!sg_is_dense(out)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_concat: out must be dense row-major");
    int64_t total = 0;
    for (int k = 0; k < n_in; ++k) {
        if ((rc = sg_validate_tensor(ctx, &in[k], "sg_concat input")) != SG_OK) return rc;
        if (in[k].rank != out->rank || in[k].dtype != out->dtype) return sg_fail(ctx, SG_ERR_SHAPE, "sg_concat: input %d rank/dtype mismatch", k);
        for (int a = 0; a < out->rank; ++a)
            if (a != axis && in[k].extents[a] != out->extents[a]) return sg_fail(ctx, SG_ERR_SHAPE, "sg_concat: not in the same shape (core.rs:848-854)");
        total += in[k].extents[axis];
    }
    if (total != out->extents[axis]) return sg_fail(ctx, SG_ERR_SHAPE, "sg_concat: extents along the axis do not add up");
    // every output element is written by exactly one input, so the reference's zero-fill is unobservable
    int64_t at = 0;
    for (int k = 0; k < n_in; ++k) {
        const sg_tensor *v = &in[k];
        const uint32_t n = (uint32_t)sg_numel(v);
        const int64_t *sets[2] = {v->strides, out->strides};
        const Dims d = collapse(v->rank, v->extents, 2, sets, -1, nullptr);
        hipLaunchKernelGGL(window_copy_kernel, dim3((n + 255) / 256), dim3(256), 0, ctx->stream, (const uint32_t *)v->base, (uint32_t *)out->base, n,
                           d, (uint32_t)v->offset, (uint32_t)(out->offset + at * out->strides[axis]));
        SG_CHECK_LAUNCH(ctx, "concat");
        at += v->extents[axis];
    }
    return SG_OK;
}

extern "C" int sg_im2col(sg_ctx *ctx, const sg_tensor *x, const sg_tensor *out, const int32_t ker[2], const int32_t stride[2],
                         const int32_t pad[2], const int32_t dil[2]) {
    if (!ctx || !ker || !stride || !pad || !dil) return SG_ERR_ARG;
    int rc;
    if ((rc = sg_validate_tensor(ctx, x, "sg_im2col x")) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, out, "sg_im2col out")) != SG_OK) return rc;
    if (x->dtype != SG_FLOAT || out->dtype != SG_FLOAT) return sg_fail(ctx, SG_ERR_DTYPE, "sg_im2col: fp32 only (conv.rs:337 reads float)");
    if (x->rank != 4 || out->rank != 6) return sg_fail(ctx, SG_ERR_SHAPE, "sg_im2col: x must be [N,H,W,C], out [N,OH,OW,KH,KW,C] (conv.rs:199)");
    if (!sg_is_dense(x) || !sg_is_dense(out)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_im2col: x and out must be dense (conv.rs:200)");
    for (int i = 0; i < 2; ++i)
        // dilation 0 is accepted: every tap then reads the same pixel, which is what the reference computes
        // (its MobileNetV2 builds such convolutions, mobilenet.rs:113)
        if (ker[i] < 1 || stride[i] < 1 || pad[i] < 0 || dil[i] < 0) return sg_fail(ctx, SG_ERR_ARG, "sg_im2col: bad geometry");
    Im2colP p;
    p.batch = (int)x->extents[0]; p.img_h = (int)x->extents[1]; p.img_w = (int)x->extents[2]; p.chan = (int)x->extents[3];
    p.ker_w = ker[0]; p.ker_h = ker[1]; p.stride_w = stride[0]; p.stride_h = stride[1];
    p.pad_w = pad[0]; p.pad_h = pad[1]; p.dil_w = dil[0]; p.dil_h = dil[1];
    // conv_size (conv.rs:47-59)
    const int64_t ow = ((int64_t)p.img_w + 2 * p.pad_w - (int64_t)p.dil_w * (p.ker_w - 1) - 1) / p.stride_w + 1;
    const int64_t oh = ((int64_t)p.img_h + 2 * p.pad_h - (int64_t)p.dil_h * (p.ker_h - 1) - 1) / p.stride_h + 1;
    if (ow < 1 || oh < 1) return sg_fail(ctx, SG_ERR_SHAPE, "sg_im2col: kernel larger than padded image");
    p.col_w = (int)ow; p.col_h = (int)oh;
    const int64_t want[6] = {p.batch, oh, ow, p.ker_h, p.ker_w, p.chan};
    for (int a = 0; a < 6; ++a)
        if (out->extents[a] != want[a]) return sg_fail(ctx, SG_ERR_SHAPE, "sg_im2col: out extent[%d] = %lld, expected %lld", a, (long long)out->extents[a], (long long)want[a]);
    const float *img = (const float *)x->base + x->offset;
    float *col = (float *)out->base + out->offset;
    const int64_t total = sg_numel(out);
    const bool vec = p.chan % 4 == 0 && ((uintptr_t)img % 16 == 0) && ((uintptr_t)col % 16 == 0);
    p.finish(vec ? 4 : 1);
    if (vec) {
        const uint32_t n = (uint32_t)(total / 4);
        hipLaunchKernelGGL((im2col_kernel<4>), dim3((n + 255) / 256), dim3(256), 0, ctx->stream, img, col, n, p);
    } else {
        const uint32_t n = (uint32_t)total;
        hipLaunchKernelGGL((im2col_kernel<1>), dim3((n + 255) / 256), dim3(256), 0, ctx->stream, img, col, n, p);
    }
    SG_CHECK_LAUNCH(ctx, "im2col");
    return SG_OK;
}

extern "C" int sg_pool2d(sg_ctx *ctx, int op, int init_mode, const sg_tensor *x, const sg_tensor *out, const int32_t ker[2],
                         const int32_t stride[2], const int32_t pad[2], const int32_t dil[2]) {
    if (!ctx || !ker || !stride || !pad || !dil) return SG_ERR_ARG;
    int rc;
    if ((rc = sg_validate_tensor(ctx, x, "sg_pool2d x")) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, out, "sg_pool2d out")) != SG_OK) return rc;
    if (op < SG_R_SUM || op > SG_R_MIN) return sg_fail(ctx, SG_ERR_ARG, "sg_pool2d: unknown op %d", op);
    if (init_mode != SG_INIT_REF_ZERO && init_mode != SG_INIT_IDENTITY) return sg_fail(ctx, SG_ERR_ARG, "sg_pool2d: bad init_mode");
    if (x->dtype != SG_FLOAT || out->dtype != SG_FLOAT) return sg_fail(ctx, SG_ERR_DTYPE, "sg_pool2d: fp32 only (conv.rs:337 reads float)");
    if (x->rank != 4 || out->rank != 4) return sg_fail(ctx, SG_ERR_SHAPE, "sg_pool2d: x must be [N,H,W,C], out [N,OH,OW,C] (conv.rs:199)");
    if (!sg_is_dense(x) || !sg_is_dense(out)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_pool2d: x and out must be dense (conv.rs:200)");
    for (int i = 0; i < 2; ++i)
        if (ker[i] < 1 || stride[i] < 1 || pad[i] < 0 || dil[i] < 0) return sg_fail(ctx, SG_ERR_ARG, "sg_pool2d: bad geometry");
    Im2colP p;
    p.batch = (int)x->extents[0]; p.img_h = (int)x->extents[1]; p.img_w = (int)x->extents[2]; p.chan = (int)x->extents[3];
    p.ker_w = ker[0]; p.ker_h = ker[1]; p.stride_w = stride[0]; p.stride_h = stride[1];
    p.pad_w = pad[0]; p.pad_h = pad[1]; p.dil_w = dil[0]; p.dil_h = dil[1];
    // conv_size (conv.rs:47-59)
    const int64_t ow = ((int64_t)p.img_w + 2 * p.pad_w - (int64_t)p.dil_w * (p.ker_w - 1) - 1) / p.stride_w + 1;
    const int64_t oh = ((int64_t)p.img_h + 2 * p.pad_h - (int64_t)p.dil_h * (p.ker_h - 1) - 1) / p.stride_h + 1;
    if (ow < 1 || oh < 1) return sg_fail(ctx, SG_ERR_SHAPE, "sg_pool2d: kernel larger than padded image");
    p.col_w = (int)ow; p.col_h = (int)oh;
    const int64_t want[4] = {p.batch, oh, ow, p.chan};
    for (int a = 0; a < 4; ++a)
        if (out->extents[a] != want[a]) return sg_fail(ctx, SG_ERR_SHAPE, "sg_pool2d: out extent[%d] = %lld, expected %lld", a, (long long)out->extents[a], (long long)want[a]);
    const float *img = (const float *)x->base + x->offset;
    float *dst = (float *)out->base + out->offset;
    const int64_t total = sg_numel(out);
    const int ref_zero = init_mode == SG_INIT_REF_ZERO;
    const bool vec = p.chan % 4 == 0 && ((uintptr_t)img % 16 == 0) && ((uintptr_t)dst % 16 == 0);
    p.finish(vec ? 4 : 1);
    if (vec) {
        const uint32_t n = (uint32_t)(total / 4);
        hipLaunchKernelGGL((pool2d_kernel<4>), dim3((n + 255) / 256), dim3(256), 0, ctx->stream, img, dst, n, p, op, ref_zero);
    } else {
        const uint32_t n = (uint32_t)total;
        hipLaunchKernelGGL((pool2d_kernel<1>), dim3((n + 255) / 256), dim3(256), 0, ctx->stream, img, dst, n, p, op, ref_zero);
    }
    SG_CHECK_LAUNCH(ctx, "pool2d");
    return SG_OK;
}

extern "C" int sg_col2im(sg_ctx *ctx, const sg_tensor *x, const sg_tensor *out, const int32_t ker[2], const int32_t stride[2],
                         const int32_t pad[2], const int32_t dil[2]) {
    if (!ctx || !ker || !stride || !pad || !dil) return SG_ERR_ARG;
    int rc;
    if ((rc = sg_validate_tensor(ctx, x, "sg_col2im x")) != SG_OK) return rc;
    if ((rc = sg_validate_tensor(ctx, out, "sg_col2im out")) != SG_OK) return rc;
    if (x->dtype != SG_FLOAT || out->dtype != SG_FLOAT) return sg_fail(ctx, SG_ERR_DTYPE, "sg_col2im: fp32 only");
    if (x->rank != 6 || out->rank != 4) return sg_fail(ctx, SG_ERR_SHAPE, "sg_col2im: x must be [N,OH,OW,KH,KW,C], out [N,H,W,C] (conv.rs:243)");
    if (!sg_is_dense(x) || !sg_is_dense(out)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_col2im: x and out must be dense (conv.rs:244)");
    for (int i = 0; i < 2; ++i)
        // dilation 0 divides by zero in the reference's kernel (conv.rs:463-465): refused
        if (ker[i] < 1 || stride[i] < 1 || pad[i] < 0 || dil[i] < 1) return sg_fail(ctx, SG_ERR_ARG, "sg_col2im: bad geometry");
    Im2colP p;
    p.batch = (int)out->extents[0]; p.img_h = (int)out->extents[1]; p.img_w = (int)out->extents[2]; p.chan = (int)out->extents[3];
    p.ker_w = ker[0]; p.ker_h = ker[1]; p.stride_w = stride[0]; p.stride_h = stride[1];
    p.pad_w = pad[0]; p.pad_h = pad[1]; p.dil_w = dil[0]; p.dil_h = dil[1];
    p.col_h = (int)x->extents[1]; p.col_w = (int)x->extents[2];
    if (x->extents[0] != p.batch || x->extents[3] != p.ker_h || x->extents[4] != p.ker_w || x->extents[5] != p.chan)
        return sg_fail(ctx, SG_ERR_SHAPE, "sg_col2im: x is not [N,OH,OW,KH,KW,C] for this kernel size and output");
    const int64_t total = sg_numel(out);
    if (total >= (1ll << 32) || sg_numel(x) >= (1ll << 32)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_col2im: more than 2^32 elements");
    const float *col = (const float *)x->base + x->offset;
    float *img = (float *)out->base + out->offset;
    const bool vec = p.chan % 4 == 0 && (uintptr_t)col % 16 == 0 && (uintptr_t)img % 16 == 0;
    p.finish(vec ? 4 : 1);
    if (vec)
        hipLaunchKernelGGL((col2im_kernel<4>), dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, ctx->stream, col, img, (uint32_t)(total / 4), p);
    else
        hipLaunchKernelGGL((col2im_kernel<1>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, col, img, (uint32_t)total, p);
    SG_CHECK_LAUNCH(ctx, "col2im");
    return SG_OK;
}
