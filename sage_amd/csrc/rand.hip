// Device random fills for gfx950: the uniform and normal generators of ops/rand.rs.
//
// Replaces Uniform::compute and Normal::compute (rand.rs:62-97, 105-146).  Both are pure functions of
// (seed_x, seed_y, element index): one xorshift128 step per sample (rand.rs:39-49) and, for the normal
// distribution, a Box-Muller transform on two consecutive samples.  The reference draws the two seeds
// from the host's thread_rng on every call (rand.rs:70, 113), so its streams are not reproducible;
// here the seeds are arguments, which is what makes the kernels testable.
#include "common.h"

namespace {

// rand.rs:39-49.  The reference's kernel text is OpenCL C built without options, where the unsuffixed literal is a
// double: the product is formed in double and rounded to float once (one seed in five gives a different last
// bit than (float)rndint * 2^-32 would).
__device__ __forceinline__ float xorshift128(uint32_t seed_x, uint32_t seed_y) {
    const uint32_t t = seed_x ^ (seed_x << 11);
    const uint32_t rndint = seed_y ^ (seed_y >> 19) ^ (t ^ (t >> 8));
    return (float)((double)rndint * 2.3283064e-10);
}

// rand.rs:77-83: y[gid] = xorshift128(seed_x + gid, seed_y + gid)
__global__ void __launch_bounds__(256) rand_uniform_kernel(float *__restrict__ y, uint32_t n, uint32_t seed_x, uint32_t seed_y) {
    const uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    if (gid < n) y[gid] = xorshift128(seed_x + gid, seed_y + gid);
}

// rand.rs:120-136: one work-item per PAIR of outputs.  The reference writes y[2 gid + 1] even when the
// element count is odd (one float past the end of its buffer); that write is dropped here.
__global__ void __launch_bounds__(256) rand_normal_kernel(float *__restrict__ y, uint32_t n, uint32_t seed_x, uint32_t seed_y) {
    const uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    if (2u * gid >= n) return;
    const float u1 = xorshift128(seed_x + gid * 2u, seed_y);
    const float u2 = xorshift128(seed_x + gid * 2u + 1u, seed_y);
    const float rsq = -2.0f * logf(u1);
    const float theta = (float)(2.0 * 3.14159265358979323846 * (double)u2);  // `2 * M_PI * u2`: M_PI is a double in OpenCL C
    const float r = sqrtf(rsq);
    y[2u * gid] = r * cosf(theta);
    if (2u * gid + 1u < n) y[2u * gid + 1u] = r * sinf(theta);
}

int check_out(sg_ctx *ctx, const sg_tensor *out, const char *who, uint32_t *n) {
    int rc = sg_validate_tensor(ctx, out, who);
    if (rc != SG_OK) return rc;
    if (out->dtype != SG_FLOAT) return sg_fail(ctx, SG_ERR_DTYPE, "%s: fp32 output (rand.rs:24, 34)", who);
    if (!sg_is_dense(out)) return sg_fail(ctx, SG_ERR_SHAPE, "%s: output must be dense", who);
    const int64_t total = sg_numel(out);
    if (total >= (1ll << 32)) return sg_fail(ctx, SG_ERR_SHAPE, "%s: more than 2^32 elements", who);
    *n = (uint32_t)total;
    return SG_OK;
}

}  // namespace

extern "C" int sg_rand_uniform(sg_ctx *ctx, uint32_t seed_x, uint32_t seed_y, const sg_tensor *out) {
    if (!ctx || !out) return SG_ERR_ARG;
    uint32_t n;
    int rc = check_out(ctx, out, "sg_rand_uniform", &n);
    if (rc != SG_OK) return rc;
    hipLaunchKernelGGL(rand_uniform_kernel, dim3((n + 255) / 256), dim3(256), 0, ctx->stream, (float *)out->base + out->offset, n, seed_x, seed_y);
    SG_CHECK_LAUNCH(ctx, "rand_uniform");
    return SG_OK;
}

extern "C" int sg_rand_normal(sg_ctx *ctx, uint32_t seed_x, uint32_t seed_y, const sg_tensor *out) {
    if (!ctx || !out) return SG_ERR_ARG;
    uint32_t n;
    int rc = check_out(ctx, out, "sg_rand_normal", &n);
    if (rc != SG_OK) return rc;
    const uint32_t pairs = (n + 1) / 2;
    hipLaunchKernelGGL(rand_normal_kernel, dim3((pairs + 255) / 256), dim3(256), 0, ctx->stream, (float *)out->base + out->offset, n, seed_x, seed_y);
    SG_CHECK_LAUNCH(ctx, "rand_normal");
    return SG_OK;
}
