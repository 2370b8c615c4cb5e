// Indexing kernels for gfx950: gather, scatter, unslice, concat, im2col, fill.
//
// These replace the reference's generated kernels of ops/core.rs (gather core.rs:674-705, scatter
// :784-819, unslice :591-600, concat :917-924) and ops/conv.rs (im2col conv.rs:304-349).  They are
// pure data movement: results are bit-exact copies.  Each thread owns consecutive output elements
// along the innermost (contiguous) output axis so stores are coalesced; coordinates come from a
// per-thread mixed-radix decomposition instead of the reference's per-axis loop of divisions, and
// im2col is parallel over every output element instead of looping batch*KH*KW inside a work-item.
#include "common.h"

namespace {

struct Dims {
    int n;
    uint32_t ext[SG_MAX_RANK];
    uint32_t stride[SG_MAX_RANK];
};

Dims dims_of(const int64_t *ext, const int64_t *st, int rank) {
    Dims d;
    d.n = rank;
    for (int i = 0; i < SG_MAX_RANK; ++i) {
        d.ext[i] = i < rank ? (uint32_t)ext[i] : 1;
        d.stride[i] = i < rank ? (uint32_t)st[i] : 0;
    }
    return d;
}

__global__ void __launch_bounds__(256) fill_u32_kernel(uint32_t *__restrict__ p, uint32_t v, uint64_t n) {
    uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    const uint64_t step = (uint64_t)gridDim.x * 256u;
    for (; i < n; i += step) p[i] = v;
}

// out[gid] = x[x_off + sum_i (i == axis ? ind[...] : c_i) * xstride_i]; c from ind's extents.
__global__ void __launch_bounds__(256) gather_kernel(const uint32_t *__restrict__ x, const uint32_t *__restrict__ ind,
                                                     uint32_t *__restrict__ y, uint32_t n, Dims idims, Dims xdims, int axis,
                                                     uint32_t x_off, uint32_t ind_off) {
    uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= n) return;
    uint32_t rem = gid, ioff = ind_off, xo = x_off, caxis_stride = xdims.stride[axis];
    for (int a = idims.n - 1; a >= 0; --a) {
        uint32_t q = rem / idims.ext[a];
        uint32_t c = rem - q * idims.ext[a];
        rem = q;
        ioff += c * idims.stride[a];
        if (a != axis) xo += c * xdims.stride[a];
    }
    const uint32_t target = ind[ioff];
    y[gid] = x[xo + target * caxis_stride];
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
    const uint32_t row = (__umulhi(gid, d_row.magic) + gid) >> d_row.shift, c = gid - row * vec_per_row;
    const uint32_t target = ind[ind_off + row * ind_row_stride];
    *reinterpret_cast<u32x4 *>(y + (size_t)gid * 4u) = *reinterpret_cast<const u32x4 *>(x + x_off + (size_t)target * x_row_stride + c * 4u);
}

template <class T>
__global__ void __launch_bounds__(256) scatter_add_kernel(const T *__restrict__ x, const uint32_t *__restrict__ ind, T *__restrict__ y,
                                                          uint32_t n, Dims idims, Dims xdims, Dims ydims, int axis, uint32_t x_off,
                                                          uint32_t ind_off) {
    uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= n) return;
    uint32_t rem = gid, ioff = ind_off, xo = x_off, yo = 0;
    for (int a = idims.n - 1; a >= 0; --a) {
        uint32_t q = rem / idims.ext[a];
        uint32_t c = rem - q * idims.ext[a];
        rem = q;
        ioff += c * idims.stride[a];
        xo += c * xdims.stride[a];
        if (a != axis) yo += c * ydims.stride[a];
    }
    yo += ind[ioff] * ydims.stride[axis];
    atomicAdd(&y[yo], x[xo]);
}

// strided window copy: y[ydims(c)] = x[xdims(c)], c enumerates x's extents
__global__ void __launch_bounds__(256) window_copy_kernel(const uint32_t *__restrict__ x, uint32_t *__restrict__ y, uint32_t n,
                                                          Dims xdims, Dims ydims, uint32_t x_off, uint32_t y_off) {
    uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= n) return;
    uint32_t rem = gid, xo = x_off, yo = y_off;
    for (int a = xdims.n - 1; a >= 0; --a) {
        uint32_t q = rem / xdims.ext[a];
        uint32_t c = rem - q * xdims.ext[a];
        rem = q;
        xo += c * xdims.stride[a];
        yo += c * ydims.stride[a];
    }
    y[yo] = x[xo];
}

struct Im2colP {
    int batch, chan, img_w, img_h, col_w, col_h, ker_w, ker_h, stride_w, stride_h, pad_w, pad_h, dil_w, dil_h;
};

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
    const uint32_t cv = p.chan / VEC;
    uint32_t rem = gid;
    const uint32_t c = (rem % cv) * VEC; rem /= cv;
    const uint32_t ox = rem % p.col_w; rem /= p.col_w;
    const uint32_t oy = rem % p.col_h; rem /= p.col_h;
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
    const uint32_t cv = p.chan / VEC;
    uint32_t rem = gid;
    uint32_t c = (rem % cv) * VEC; rem /= cv;
    uint32_t kx = rem % p.ker_w; rem /= p.ker_w;
    uint32_t ky = rem % p.ker_h; rem /= p.ker_h;
    uint32_t ox = rem % p.col_w; rem /= p.col_w;
    uint32_t oy = rem % p.col_h; rem /= p.col_h;
    uint32_t n = rem;
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

// Col2im::compute (conv.rs:405-500): img[n,y,x,c] = sum of the column entries that im2col copied
// from that pixel.  One thread per output element (the reference loops the batch inside a work-item);
// the additions run col_x outer, col_y inner, as the reference's, so the sum is bit-identical to a
// sequential restatement.  The reference tests ker_x against dilation_h and ker_y against dilation_w
// (conv.rs:463-465); kept, it only matters when the two dilations differ.
// VEC = 4: a thread sums four consecutive channels (16-byte loads, one 16-byte store); each channel's additions
// keep their order.
template <int VEC>
__global__ void __launch_bounds__(256) col2im_kernel(const float *__restrict__ col, float *__restrict__ img, uint32_t n_out, Im2colP p) {
    typedef float vec_t __attribute__((ext_vector_type(VEC)));
    const uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= n_out) return;
    const uint32_t cv = p.chan / VEC;  // channel groups per pixel
    const int c = (gid % cv) * VEC;
    uint32_t t = gid / cv;
    const int img_x = t % p.img_w;
    t /= p.img_w;
    const int img_y = t % p.img_h;
    const int n = t / p.img_h;
    const int img_x_pad = img_x + p.pad_w, img_y_pad = img_y + p.pad_h;
    const int ker_ew = (p.ker_w - 1) * p.dil_w + 1, ker_eh = (p.ker_h - 1) * p.dil_h + 1;
    const int col_x_start = img_x_pad < ker_ew ? 0 : (img_x_pad - ker_ew) / p.stride_w + 1;
    const int col_y_start = img_y_pad < ker_eh ? 0 : (img_y_pad - ker_eh) / p.stride_h + 1;
    const int col_x_end = min(img_x_pad / p.stride_w + 1, p.col_w);
    const int col_y_end = min(img_y_pad / p.stride_h + 1, p.col_h);
    const float *cb = col + (size_t)n * p.col_h * p.col_w * p.ker_h * p.ker_w * p.chan + c;
    vec_t val = 0.0f;
    for (int col_x = col_x_start; col_x < col_x_end; ++col_x)
        for (int col_y = col_y_start; col_y < col_y_end; ++col_y) {
            int ker_x = img_x_pad - col_x * p.stride_w, ker_y = img_y_pad - col_y * p.stride_h;
            if (ker_x % p.dil_h == 0 && ker_y % p.dil_w == 0) {
                ker_x /= p.dil_h;
                ker_y /= p.dil_w;
                val += *reinterpret_cast<const vec_t *>(cb + (size_t)(((col_y * p.col_w + col_x) * p.ker_h + ker_y) * p.ker_w + ker_x) * p.chan);
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
    Dims idims = dims_of(ind->extents, ind->strides, ind->rank), xdims = dims_of(x->extents, x->strides, x->rank);
    hipLaunchKernelGGL(gather_kernel, dim3((n + 255) / 256), dim3(256), 0, ctx->stream, (const uint32_t *)x->base, (const uint32_t *)ind->base,
                       (uint32_t *)out->base + out->offset, n, idims, xdims, axis, (uint32_t)x->offset, (uint32_t)ind->offset);
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
    Dims idims = dims_of(ind->extents, ind->strides, ind->rank), xdims = dims_of(x->extents, x->strides, x->rank),
         ydims = dims_of(out->extents, out->strides, out->rank);
    dim3 grid((n + 255) / 256);
    if (x->dtype == SG_FLOAT)
        hipLaunchKernelGGL((scatter_add_kernel<float>), grid, dim3(256), 0, ctx->stream, (const float *)x->base, (const uint32_t *)ind->base,
                           (float *)out->base + out->offset, n, idims, xdims, ydims, axis, (uint32_t)x->offset, (uint32_t)ind->offset);
    else
        hipLaunchKernelGGL((scatter_add_kernel<unsigned>), grid, dim3(256), 0, ctx->stream, (const unsigned *)x->base, (const uint32_t *)ind->base,
                           (unsigned *)out->base + out->offset, n, idims, xdims, ydims, axis, (uint32_t)x->offset, (uint32_t)ind->offset);
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
    Dims xdims = dims_of(x->extents, x->strides, x->rank), ydims = dims_of(x->extents, out->strides, x->rank);
    hipLaunchKernelGGL(window_copy_kernel, dim3((n + 255) / 256), dim3(256), 0, ctx->stream, (const uint32_t *)x->base, (uint32_t *)out->base, n,
                       xdims, ydims, (uint32_t)x->offset, (uint32_t)(out->offset + start * out->strides[axis]));
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
        Dims xdims = dims_of(v->extents, v->strides, v->rank), ydims = dims_of(v->extents, out->strides, v->rank);
        hipLaunchKernelGGL(window_copy_kernel, dim3((n + 255) / 256), dim3(256), 0, ctx->stream, (const uint32_t *)v->base, (uint32_t *)out->base, n,
                           xdims, ydims, (uint32_t)v->offset, (uint32_t)(out->offset + at * out->strides[axis]));
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
        // dilation 0 would divide by zero in the reference's kernel (conv.rs:463-465): refused
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
    if (p.chan % 4 == 0 && (uintptr_t)col % 16 == 0 && (uintptr_t)img % 16 == 0)
        hipLaunchKernelGGL((col2im_kernel<4>), dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, ctx->stream, col, img, (uint32_t)(total / 4), p);
    else
        hipLaunchKernelGGL((col2im_kernel<1>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, col, img, (uint32_t)total, p);
    SG_CHECK_LAUNCH(ctx, "col2im");
    return SG_OK;
}
