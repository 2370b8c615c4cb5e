// One Adam step over many parameters in one launch, in place, for gfx950.
//
// Adam::update (optim.rs:129-177) builds, per parameter, three map operators (new first moment, new
// second moment, new value) out of about twenty scalar ones and evaluates them one parameter after
// the other; replaying that as launches costs six per parameter (three kernels, three copies into the
// persistent buffers): 252 launches of a few microseconds for the 42 parameters of ResNet-18, more
// than the backward pass itself.  Here up to 32 parameters share a launch: a workgroup finds its
// tensor in a table passed by value and every thread rewrites four pieces of four consecutive elements
// of the two moments and the value (the two powers of beta, the costly part, are formed once per thread).
//
// The arithmetic is the reference's expression, operation for operation and without contraction
// (this file is compiled with -ffp-contract=off, like the generated map kernels), so the result is
// bit-identical to the operator chain:
//   g  = grad (+ value * weight_decay, when weight_decay != 0)              optim.rs:138-142
//   m' = m * beta1 + g * (1 - beta1)                                        optim.rs:149-155
//   v' = v * beta2 + pow(g, 2) * (1 - beta2)                                optim.rs:157-163
//   value' = value - (m' / (-pow(beta1, t) + 1)) * lr / (sqrt(v' / (-pow(beta2, t) + 1)) + eps)   optim.rs:165-174
// with t read from device memory (the reference keeps it as a tensor and adds 1 per update).
#include "common.h"

namespace {

constexpr int ADAM_MAX = 32;      // tensors per launch
constexpr int ADAM_BLOCK = 4096;  // elements per workgroup: 256 threads x 4 pieces of 4

struct AdamTensor {
    float *value;
    const float *grad;
    float *m, *v;
    uint32_t n;            // elements
    uint32_t first_block;  // index of this tensor's first workgroup
    uint32_t vec;          // all four pointers 16-byte aligned
};

struct AdamArgs {
    AdamTensor t[ADAM_MAX];
    int count;
    const float *step;
    float lr, beta1, beta2, one_minus_beta1, one_minus_beta2, eps, weight_decay;
};

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void adam_element(float &value, float g0, float &m, float &v, const AdamArgs &a, float den1, float den2) {
    const float g = a.weight_decay != 0.0f ? g0 + value * a.weight_decay : g0;
    m = m * a.beta1 + g * a.one_minus_beta1;
    v = v * a.beta2 + powf(g, 2.0f) * a.one_minus_beta2;
    const float m_hat = m / den1;
    const float v_hat = v / den2;
    value = value - m_hat * a.lr / (sqrtf(v_hat) + a.eps);
}

__global__ void __launch_bounds__(256) adam_kernel(const AdamArgs a) {
    // the table is ordered by first_block: the last entry that starts at or before this workgroup
    int k = 0;
    for (int i = 1; i < a.count; ++i)
        if (a.t[i].first_block <= blockIdx.x) k = i;
    const AdamTensor t = a.t[k];
    const uint32_t base = (blockIdx.x - t.first_block) * ADAM_BLOCK + threadIdx.x * 4u;
    if (base >= t.n) return;
    const float step = *a.step;
    const float den1 = -powf(a.beta1, step) + 1.0f, den2 = -powf(a.beta2, step) + 1.0f;
    for (uint32_t i0 = base; i0 < t.n && i0 < base + ADAM_BLOCK; i0 += 1024u) {
        if (t.vec && i0 + 4 <= t.n) {
            const f32x4 p4 = *reinterpret_cast<const f32x4 *>(t.value + i0), g4 = *reinterpret_cast<const f32x4 *>(t.grad + i0);
            const f32x4 m4 = *reinterpret_cast<const f32x4 *>(t.m + i0), v4 = *reinterpret_cast<const f32x4 *>(t.v + i0);
            float p[4] = {p4.x, p4.y, p4.z, p4.w}, m[4] = {m4.x, m4.y, m4.z, m4.w}, v[4] = {v4.x, v4.y, v4.z, v4.w};
            const float g[4] = {g4.x, g4.y, g4.z, g4.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) adam_element(p[j], g[j], m[j], v[j], a, den1, den2);
            *reinterpret_cast<f32x4 *>(t.m + i0) = f32x4{m[0], m[1], m[2], m[3]};
            *reinterpret_cast<f32x4 *>(t.v + i0) = f32x4{v[0], v[1], v[2], v[3]};
            *reinterpret_cast<f32x4 *>(t.value + i0) = f32x4{p[0], p[1], p[2], p[3]};
        } else {
            const uint32_t i1 = i0 + 4 < t.n ? i0 + 4 : t.n;
            for (uint32_t i = i0; i < i1; ++i) {
                float p = t.value[i], m = t.m[i], v = t.v[i];
                adam_element(p, t.grad[i], m, v, a, den1, den2);
                t.m[i] = m;
                t.v[i] = v;
                t.value[i] = p;
            }
        }
    }
}

bool aligned16(const float *p) { return ((uintptr_t)p) % 16 == 0; }

int dense_f32(sg_ctx *ctx, const sg_tensor *t, const char *who, int64_t *n) {
    int rc = sg_validate_tensor(ctx, t, who);
    if (rc != SG_OK) return rc;
    if (t->dtype != SG_FLOAT) return sg_fail(ctx, SG_ERR_DTYPE, "%s: fp32 only", who);
    if (!sg_is_dense(t)) return sg_fail(ctx, SG_ERR_SHAPE, "%s: must be dense row-major", who);
    *n = sg_numel(t);
    return SG_OK;
}

}  // namespace

extern "C" int sg_adam_update(sg_ctx *ctx, int n_tensors, const sg_tensor *values, const sg_tensor *grads, const sg_tensor *m,
                              const sg_tensor *v, const sg_tensor *step, const sg_adam_hyper *h) {
    if (!ctx || n_tensors < 0 || (n_tensors && (!values || !grads || !m || !v)) || !step || !h) return SG_ERR_ARG;
    int rc;
    int64_t n_step = 0;
    if ((rc = dense_f32(ctx, step, "sg_adam_update step", &n_step)) != SG_OK) return rc;
    if (n_step != 1) return sg_fail(ctx, SG_ERR_SHAPE, "sg_adam_update step: one element expected");
    // validate everything before the first launch: a failed call changes nothing
    for (int i = 0; i < n_tensors; ++i) {
        int64_t n = 0, ng = 0, nm = 0, nv = 0;
        if ((rc = dense_f32(ctx, &values[i], "sg_adam_update value", &n)) != SG_OK) return rc;
        if ((rc = dense_f32(ctx, &grads[i], "sg_adam_update grad", &ng)) != SG_OK) return rc;
        if ((rc = dense_f32(ctx, &m[i], "sg_adam_update first moment", &nm)) != SG_OK) return rc;
        if ((rc = dense_f32(ctx, &v[i], "sg_adam_update second moment", &nv)) != SG_OK) return rc;
        if (ng != n || nm != n || nv != n) return sg_fail(ctx, SG_ERR_SHAPE, "sg_adam_update: tensor %d: value, gradient and moments differ in size", i);
        if (n >= (1ll << 31)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_adam_update: tensor %d: more than 2^31 elements", i);
    }
    for (int first = 0; first < n_tensors; first += ADAM_MAX) {
        AdamArgs a{};
        a.step = (const float *)step->base + step->offset;
        a.lr = h->lr; a.beta1 = h->beta1; a.beta2 = h->beta2; a.one_minus_beta1 = h->one_minus_beta1; a.one_minus_beta2 = h->one_minus_beta2;
        a.eps = h->eps; a.weight_decay = h->weight_decay;
        uint64_t blocks = 0;
        for (int i = first; i < n_tensors && i < first + ADAM_MAX; ++i) {
            const int64_t n = sg_numel(&values[i]);
            if (n == 0) continue;
            AdamTensor &t = a.t[a.count++];
            t.value = (float *)values[i].base + values[i].offset;
            t.grad = (const float *)grads[i].base + grads[i].offset;
            t.m = (float *)m[i].base + m[i].offset;
            t.v = (float *)v[i].base + v[i].offset;
            t.n = (uint32_t)n;
            t.first_block = (uint32_t)blocks;
            t.vec = aligned16(t.value) && aligned16(t.grad) && aligned16(t.m) && aligned16(t.v);
            blocks += (uint64_t)(n + ADAM_BLOCK - 1) / ADAM_BLOCK;
        }
        if (a.count == 0) continue;
        if (blocks >= (1ull << 31)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_adam_update: too many elements for one launch");
        hipLaunchKernelGGL(adam_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, a);
        SG_CHECK_LAUNCH(ctx, "adam");
    }
    return SG_OK;
}
