/*
 * sage_hip.h — C ABI of the MI355X (gfx950) compute backend for Sage's operator hot path.
 *
 * Every entry point replaces one device-side responsibility of the reference (ingim/sage); the
 * reference interface it stands in for is cited as file:line under the reference's `src/`.
 * The boundary is the operator `compute` call (ops.rs:79-101, dispatched from ops.rs:163-187):
 * strided tensor descriptors in, a freshly written contiguous tensor out, status-code errors.
 *
 * Conventions
 *  - Plain C: pointers, sizes, PODs.  No C++ or torch types cross this boundary.
 *  - Every function returns an sg_status.  Nothing aborts; after a non-OK return
 *    sg_last_error() describes it, and for SG_ERR_OOM sg_last_oom() gives {needed,total}
 *    (error.rs:5-13, session/memory.rs:45-54).
 *  - A context owns one device, one in-order HIP stream, the kernel cache and the allocator
 *    (session/context.rs:25-52).  Launches are asynchronous on that stream; sg_memcpy_d2h and
 *    sg_sync wait for it (session/device.rs:111-147 are blocking the same way).
 *  - A context is not thread-safe (the reference threads `&mut Context` everywhere); distinct
 *    contexts are independent.
 *  - The library never frees or reallocates caller memory.  Outputs are allocated by the caller
 *    with sg_alloc and passed in; op outputs must be dense row-major ("default strides",
 *    shape.rs:45-54) at any element offset, as the reference's outputs are (tensor.rs:195-210).
 *  - Strides and offsets count ELEMENTS, not bytes; stride 0 is a broadcast axis
 *    (shape.rs:190-195, 239-279).  Index arithmetic is exact.
 *  - Only 4-byte element types are computed on (SG_FLOAT, SG_INT, SG_UINT): the reference sizes
 *    every buffer as numel*4 bytes (session/device.rs:75), so nothing else is safe there either.
 *    Other dtypes yield SG_ERR_DTYPE.
 */
#ifndef SAGE_HIP_H
#define SAGE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SG_MAX_RANK 8
#define SG_MAX_MAP_INPUTS 16
#define SG_MAX_EXPR 128
/* Allocator capacity a default reference Context runs with: 1000 MiB (session/context.rs:49). */
#define SG_REFERENCE_CAPACITY_BYTES (1000ull * 1024ull * 1024ull)

typedef enum sg_status {
    SG_OK = 0,
    SG_ERR_OOM = 1,    /* Error::Memory(OutOfMemory{mem_needed,mem_total})  memory.rs:246-255 */
    SG_ERR_DEVICE = 2, /* Error::Device(ocl::Error) -> a hipError_t / hiprtc failure          */
    SG_ERR_SHAPE = 3,  /* Error::Shape / the reference's shape assert!/panic! sites            */
    SG_ERR_DTYPE = 4,  /* the reference's dtype assert_eq! sites (map.rs:489, 869-870)         */
    SG_ERR_ARG = 5     /* null pointer, bad enum, unsupported combination                      */
} sg_status;

/* Same order as the reference's DataType enum (tensor/data.rs:14-30). */
typedef enum sg_dtype {
    SG_CHAR = 0, SG_SHORT = 1, SG_INT = 2, SG_LONG = 3,
    SG_UCHAR = 4, SG_USHORT = 5, SG_UINT = 6, SG_ULONG = 7,
    SG_FLOAT = 8, SG_HALF = 9
} sg_dtype;

/* TensorDesc + Shape (tensor.rs:38-41, shape.rs:38-42) plus the device pointer of the buffer. */
typedef struct sg_tensor {
    void *base;                   /* device pointer of element 0 of the underlying buffer */
    int32_t dtype;                /* sg_dtype */
    int32_t rank;                 /* 1..SG_MAX_RANK */
    int64_t extents[SG_MAX_RANK];
    int64_t strides[SG_MAX_RANK]; /* elements; 0 = broadcast */
    int64_t offset;               /* elements */
} sg_tensor;

typedef struct sg_ctx sg_ctx;

/* ---- context, memory, transfers: session/context.rs:43-52, session/device.rs:45-191 ---------- */

/* Context::with_device (context.rs:43-52) + Device::new (device.rs:45-70).  capacity_bytes bounds
 * the bytes handed out by sg_alloc (Allocator::new capacity, memory.rs:173-180); 0 = no cap beyond
 * the device.  The reference default is SG_REFERENCE_CAPACITY_BYTES. */
int sg_ctx_create(int device_idx, uint64_t capacity_bytes, sg_ctx **out);
/* The same with the allocator's two switches, Allocator::new(capacity, use_cache, use_sub_buffer) (memory.rs:64-69,
 * 224-236).  use_cache = 0 is sg_ctx_create (what the reference's Context builds, context.rs:49).  use_cache = 1
 * takes memory from the device in chunks and serves requests from them, Pool::alloc's caching branch
 * (memory.rs:262-352, 364-475): requests below 1 MiB from 2 MiB chunks, larger ones from 20 MiB chunks, requests
 * of 10 MiB and more from chunks of their own size rounded up to 2 MiB (allocation_size, memory.rs:257-265); the
 * smallest free block that fits and is not wastefully large (a request below 40 MiB never takes a block of 40 MiB
 * or more, a larger one never a block 20 MiB beyond its size), split when the rest is worth keeping (>= 512 B
 * behind a request up to 1 MiB, > 1 MiB behind one below 40 MiB; use_sub_buffer = 0: never split), neighbours of
 * one chunk merged again when freed; when nothing fits: whole free chunks older than the average age are returned
 * to the device once 80 % of the capacity is in use, a new chunk is taken, and if the capacity forbids that the
 * largest whole free chunks of the large class are returned first (then, beyond the reference, those of the small
 * class).  Sizes are rounded up to 256 B so that every block keeps the
 * alignment of a device allocation.  sg_mem_stats then reports used = bytes of the blocks handed out, reserved =
 * bytes of the chunks held (the figure the capacity bounds, Pool::check_space), peak = the most ever held. */
int sg_ctx_create_pooled(int device_idx, uint64_t capacity_bytes, int use_cache, int use_sub_buffer, sg_ctx **out);
int sg_ctx_destroy(sg_ctx *ctx);

/* Context::alloc -> Pool::alloc -> Device::alloc_buffer (context.rs:119-137, memory.rs:353-362,
 * device.rs:73-89).  Over-capacity -> SG_ERR_OOM with needed = (total+size)-capacity,
 * total = bytes currently reserved (memory.rs:246-255).  Freed blocks are cached and reused on the
 * context's single in-order stream; sg_trim returns the cache to the device. */
int sg_alloc(sg_ctx *ctx, uint64_t nbytes, void **dptr);
/* OpenClMemory::drop (memory.rs:685-692). */
int sg_free(sg_ctx *ctx, void *dptr);
int sg_trim(sg_ctx *ctx);
/* Allocator::{mem_used,mem_total,mem_peak,capacity} (memory.rs:182-198), in bytes. */
int sg_mem_stats(sg_ctx *ctx, uint64_t *used, uint64_t *reserved, uint64_t *peak, uint64_t *capacity);

/* Buffer::write / Buffer::read (device.rs:111-147): blocking copies. */
int sg_memcpy_h2d(sg_ctx *ctx, void *dst_dev, const void *src_host, uint64_t nbytes);
int sg_memcpy_d2h(sg_ctx *ctx, void *dst_host, const void *src_dev, uint64_t nbytes);
int sg_memcpy_d2d(sg_ctx *ctx, void *dst_dev, const void *src_dev, uint64_t nbytes);
/* Buffer::fill (device.rs:149-164) as used by Tensor::fill_zero (tensor.rs:212): 32-bit pattern. */
int sg_fill_u32(sg_ctx *ctx, void *dst_dev, uint32_t pattern, uint64_t count);
/* Queue::finish.  sg_stream returns the context's hipStream_t so a caller can time with events. */
int sg_sync(sg_ctx *ctx);
void *sg_stream(sg_ctx *ctx);

/* Device-side timing on the context's stream.  The reference only wall-clocks a routine on the
 * host (Routine::exec, session.rs:619, 667-668); these wrap hipEvent so a caller can time the
 * launches it issued between two records. */
int sg_event_create(sg_ctx *ctx, void **event);
int sg_event_record(sg_ctx *ctx, void *event);
int sg_event_elapsed_ms(sg_ctx *ctx, void *start, void *stop, float *ms);
int sg_event_destroy(sg_ctx *ctx, void *event);

const char *sg_last_error(sg_ctx *ctx);
int sg_last_oom(sg_ctx *ctx, uint64_t *needed, uint64_t *total);
/* Number of distinct kernels built at run time so far (Context::kernels, context.rs:29-31). */
int sg_kernel_cache_size(sg_ctx *ctx);

/* ---- fused elementwise maps: ops/map.rs ------------------------------------------------------ */

/* UnaryMap (map.rs:93-130), BinaryMap (map.rs:152-172), TernaryMap (map.rs:194-196): same order. */
typedef enum sg_unary {
    SG_U_COPY = 0, SG_U_ABS, SG_U_NEG, SG_U_RECIP, SG_U_LOG, SG_U_EXP, SG_U_SQRT, SG_U_SQUARE,
    SG_U_ERF, SG_U_SIGN, SG_U_CEIL, SG_U_FLOOR, SG_U_ROUND,
    SG_U_SIN, SG_U_SINH, SG_U_COS, SG_U_COSH, SG_U_TAN, SG_U_TANH,
    SG_U_ASIN, SG_U_ASINH, SG_U_ACOS, SG_U_ACOSH, SG_U_ATAN, SG_U_ATANH,
    SG_U_NOT, SG_U_CAST_INT, SG_U_CAST_FLOAT, SG_U__COUNT
} sg_unary;
typedef enum sg_binary {
    SG_B_ADD = 0, SG_B_SUB, SG_B_DIV, SG_B_MUL, SG_B_MOD, SG_B_POW, SG_B_MIN, SG_B_MAX,
    SG_B_AND, SG_B_OR, SG_B_EQ, SG_B_NE, SG_B_GT, SG_B_GE, SG_B_LT, SG_B_LE, SG_B__COUNT
} sg_binary;
typedef enum sg_ternary { SG_T_COND = 0, SG_T__COUNT } sg_ternary;

typedef enum sg_expr_kind {
    SG_EXPR_INPUT = 0,   /* StackElement::Input(idx)              map.rs:218-222 */
    SG_EXPR_LITERAL = 1, /* NullaryMap::Literal  "(type)value"     map.rs:517-531 */
    SG_EXPR_UNARY = 2,
    SG_EXPR_BINARY = 3,
    SG_EXPR_TERNARY = 4
} sg_expr_kind;

/* One element of VariadicMapOperator.expr (map.rs:199-222) in the same PREFIX order the reference
 * stores it: an operator is followed by its operands, left to right (ops.rs:116-130). */
typedef struct sg_expr {
    int32_t kind;  /* sg_expr_kind */
    int32_t op;    /* sg_unary / sg_binary / sg_ternary, or the input index for SG_EXPR_INPUT */
    int32_t dtype; /* SG_EXPR_LITERAL: sg_dtype of the literal (SG_FLOAT, SG_INT or SG_UINT) */
    uint32_t bits; /* SG_EXPR_LITERAL: the 32-bit pattern of the value */
} sg_expr;

/* {Nullary,Unary,Binary,Ternary,Variadic}MapOperator::compute via compile_map (map.rs:369-410,
 * 898-921, 970-998, 1044-1078, 1101-1120, 1141-1175): out[gid] = expr(in_0[idx_0], ...), with idx_i
 * from translate_id (core.rs:113-175).  All inputs must have out's extents (the reference
 * broadcasts beforehand with Expand -> stride 0, map.rs:412-456).  Result dtype follows
 * map.rs:464-470, 491-501 and is checked against out->dtype.  n_in may be 0 (nullary_map).
 * SG_B_MOD returns SG_ERR_ARG: the reference emits `mod(a, b)`, which is not an OpenCL C function,
 * so its kernel cannot be built either (map.rs:275; its test is disabled, map.rs:1603). */
int sg_map(sg_ctx *ctx, const sg_expr *prog, int n_prog, const sg_tensor *in, int n_in,
           const sg_tensor *out);
/* The kernel text sg_map would build for these operands (compile_map's return value,
 * map.rs:369-410), without building or launching it; base pointers may be null.  Writes at most
 * cap-1 bytes plus a terminator, and the dtype the expression yields.  ctx may be null. */
int sg_map_source(sg_ctx *ctx, const sg_expr *prog, int n_prog, const sg_tensor *in, int n_in,
                  const sg_tensor *out, char *buf, uint64_t cap, int32_t *result_dtype);
/* Compiles kernel text for gfx950 exactly as sg_map does (KernelProgram::new, device.rs:201-213)
 * but loads nothing, so it needs no GPU.  On failure the build log goes to log_buf. */
int sg_map_compile_only(const char *source, char *log_buf, uint64_t log_cap);

/* ---- reductions: ops/reduce.rs --------------------------------------------------------------- */

typedef enum sg_reduce_op { SG_R_SUM = 0, SG_R_PROD = 1, SG_R_MAX = 2, SG_R_MIN = 3 } sg_reduce_op;
typedef enum sg_reduce_arg_op { SG_RA_MAX = 0, SG_RA_MIN = 1 } sg_reduce_arg_op;
/* The reference starts every accumulator at literal 0 (reduce.rs:282), so its max is
 * max(0, true max), its min is min(0, true min) and its prod is 0.  SG_INIT_REF_ZERO reproduces
 * that bit for bit; SG_INIT_IDENTITY uses -inf/+inf/1/0.  Sum is identical under both. */
typedef enum sg_reduce_init { SG_INIT_REF_ZERO = 0, SG_INIT_IDENTITY = 1 } sg_reduce_init;

/* ReduceOperator::compute (reduce.rs:258-325).  `out` extents must be reduced_extents(in, axes,
 * preserve) for either value of preserve (reduce.rs:124-140): only numel and contiguity matter. */
int sg_reduce(sg_ctx *ctx, int op, const int32_t *axes, int n_axes, int init_mode,
              const sg_tensor *in, const sg_tensor *out);
/* ReduceArgOperator::compute (reduce.rs:372-431): first extreme index wins ties; out is SG_UINT. */
int sg_reduce_arg(sg_ctx *ctx, int op, int axis, const sg_tensor *in, const sg_tensor *out);

/* ---- indexing kernels: ops/core.rs ----------------------------------------------------------- */

/* Gather::compute (core.rs:655-718): out has ind's extents; ind is SG_UINT or SG_INT read as
 * unsigned (core.rs:679) through its own strides (stride 0 allowed).  No bounds check on the
 * reference; here an index >= x.extents[axis] is not detected either (caller's contract). */
int sg_gather(sg_ctx *ctx, int axis, const sg_tensor *x, const sg_tensor *ind, const sg_tensor *out);
/* Scatter::compute (core.rs:764-833): out is zero-filled, then out[.., ind, ..] += x.  The
 * reference's update is a non-atomic read-modify-write, so duplicate indices race there; here the
 * add is atomic (deterministic up to fp32 summation order).  ind must have default strides: the
 * reference decomposes gid by ind's own strides (core.rs:770, 807-808). */
int sg_scatter(sg_ctx *ctx, int axis, const sg_tensor *x, const sg_tensor *ind, const sg_tensor *out);
/* Unslice::compute (core.rs:553-611): out zero-filled, x copied into [start, start+x.extents[axis]). */
int sg_unslice(sg_ctx *ctx, int axis, int64_t start, const sg_tensor *x, const sg_tensor *out);
/* Concat::compute (core.rs:892-934). */
int sg_concat(sg_ctx *ctx, int axis, const sg_tensor *in, int n_in, const sg_tensor *out);

/* ---- GEMM: ops/gemm.rs + ops/kernels/matmul_direct.opencl ------------------------------------ */

typedef enum sg_act { SG_ACT_NONE = 0, SG_ACT_RELU = 1, SG_ACT_GELU_ERF = 2 } sg_act;

/* Optional fused epilogue (no counterpart in the reference, which runs each of these as a separate
 * full-size map launch after the GEMM: layers.rs:243-247, nn.rs:33-40, bert.rs:203,279):
 *   v = alpha * (A.B)[m,n];  v += bias[n];  v = act(v);  v += residual[m,n];  v = act_post(v).
 * A null sg_gemm_epilogue* means alpha = 1 and nothing else, i.e. exactly the reference's GEMM
 * (alpha = 1, beta = 0, gemm.rs:227-228). */
typedef struct sg_gemm_epilogue {
    float alpha;
    int32_t act;               /* sg_act, applied after bias */
    int32_t act_post;          /* sg_act, applied after residual */
    const sg_tensor *bias;     /* numel == N, unit stride, or NULL */
    const sg_tensor *residual; /* [M,N], [batch,M,N] (batch axes flattened) or C's extents; last stride 1; or NULL */
} sg_gemm_epilogue;

/* (A long-K product with few output tiles uses a workspace from the context allocator: SG_ERR_OOM when it does not fit.)
 * Gemm::compute_direct (gemm.rs:176-250): a, b, c are rank 2; (m,k,n) are taken from the extents
 * as gemm.rs:190-217 does for the four transpose modes; ld = strides[0] and the inner stride must
 * be 1 (the reference organizes its inputs first, gemm.rs:111-112).  fp32 only. */
int sg_gemm(sg_ctx *ctx, int transpose_a, int transpose_b, const sg_tensor *a, const sg_tensor *b,
            const sg_tensor *c, const sg_gemm_epilogue *epi);
/* No counterpart in the reference.  For callers that cannot allocate device memory at the call:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same
 * arguments, same kernels and bit-identical results as sg_gemm, but the split-K workspace of a
 * few-tile/long-K product is a static array of SG_GEMM_NOALLOC_SCRATCH_BYTES in the library's code
 * object (one copy per GPU, held until the process ends) instead of a block from the context's
 * allocator; the call performs no allocation or free of any kind.  A product whose split-K partial
 * products (ranges x M x N x 4 bytes) exceed the array returns SG_ERR_ARG and computes nothing.
 * All contexts on one GPU share that GPU's array: calls that may overlap on one GPU (different
 * contexts/streams, or two replays of graphs holding this call) race and must be serialised by
 * the caller.  Nothing in the array needs clearing between calls: pass 1 overwrites every element
 * pass 2 reads. */
#define SG_GEMM_NOALLOC_SCRATCH_BYTES (32u << 20)
int sg_gemm_noalloc(sg_ctx *ctx, int transpose_a, int transpose_b, const sg_tensor *a,
                    const sg_tensor *b, const sg_tensor *c, const sg_gemm_epilogue *epi);
/* GemmBatched::compute_direct (gemm.rs:338-421): rank 3, batch stride = strides[0], ld = strides[1]. */
int sg_gemm_batched(sg_ctx *ctx, int transpose_a, int transpose_b, const sg_tensor *a,
                    const sg_tensor *b, const sg_tensor *c, const sg_gemm_epilogue *epi);
/* matmul_batched (gemm.rs:53-104) without its organize copies: a = [batch.., M, K],
 * b = [batch.., K, N], c = [batch.., M, N] with up to two leading batch axes and arbitrary strides,
 * provided each matrix has one unit stride among its two inner axes (c: the N axis).  This is how
 * permuted attention heads (bert.rs:282-302) are consumed and produced in place. */
int sg_matmul_strided(sg_ctx *ctx, const sg_tensor *a, const sg_tensor *b, const sg_tensor *c,
                      const sg_gemm_epilogue *epi);

/* Name of the kernel instantiation the most recent product on this context launched (sg_gemm,
 * sg_gemm_batched, sg_matmul_strided, sg_conv2d; for a split-K product: its first pass), as it appears
 * in a rocprofv3 kernel trace: tile sizes, operand layouts, guarded loads, image addressing and the kind of
 * write-out are template arguments.  The reference has one fixed 8x8 kernel per transpose mode (gemm.rs:208-221);
 * here the instantiation is chosen per shape.  SG_ERR_ARG before the first product. */
int sg_gemm_last_kernel_name(sg_ctx *ctx, char *buf, uint64_t cap);

/* ---- convolution feeder: ops/conv.rs --------------------------------------------------------- */

/* Im2col::compute (conv.rs:289-374): x [N,H,W,C] dense -> out [N,OH,OW,KH,KW,C], zero padding.
 * Every pair is {w, h} as in the reference (conv.rs:83, 205-206). */
int sg_im2col(sg_ctx *ctx, const sg_tensor *x, const sg_tensor *out, const int32_t ker[2],
              const int32_t stride[2], const int32_t pad[2], const int32_t dil[2]);

/* conv_2d (conv.rs:61-96) in one launch: out[N,OH,OW,OC] = im2col(x)[N*OH*OW, KH*KW*C] . filter[KH*KW*C, OC]
 * with the column matrix never written (the reference launches Im2col::compute, conv.rs:289-374, and then
 * Gemm::compute_direct on its output).  x [N,H,W,C], filter [KH,KW,C,OC], out dense; pairs are {w, h};
 * the kernel size comes from the filter.  epi as in sg_gemm (bias over OC, residual as [N*OH*OW, OC]:
 * the output seen as a matrix).  A few-tile/long-K product uses a split-K workspace from the context allocator (SG_ERR_OOM). */
int sg_conv2d(sg_ctx *ctx, const sg_tensor *x, const sg_tensor *filter, const sg_tensor *out,
              const int32_t stride[2], const int32_t pad[2], const int32_t dil[2],
              const sg_gemm_epilogue *epi);

/* max_pool_2d / avg_pool_2d (conv.rs:143-165) without the column tensor: out[N,OH,OW,C] = reduce over the
 * kernel window of x[N,H,W,C], exactly what Im2col::compute (conv.rs:289-374) followed by
 * ReduceOperator::compute over axes [3,4] (reduce.rs:258-325) gives: pixels outside the image count as
 * zeros, op and init_mode as in sg_reduce (avg_pool divides the SUM by the window size afterwards). */
int sg_pool2d(sg_ctx *ctx, int op, int init_mode, const sg_tensor *x, const sg_tensor *out,
              const int32_t ker[2], const int32_t stride[2], const int32_t pad[2], const int32_t dil[2]);

/* Col2im::compute (conv.rs:405-500), the adjoint of sg_im2col used by Im2col::grad (conv.rs:275-287):
 * x [N,OH,OW,KH,KW,C] dense -> out [N,H,W,C], each pixel the sum of the column entries taken from
 * it (additions in the reference's order: column x outer, column y inner). */
int sg_col2im(sg_ctx *ctx, const sg_tensor *x, const sg_tensor *out, const int32_t ker[2],
              const int32_t stride[2], const int32_t pad[2], const int32_t dil[2]);

/* ---- random fills: ops/rand.rs ------------------------------------------------------------- */

/* Uniform::compute (rand.rs:62-97): out[i] = xorshift128(seed_x + i, seed_y + i) in [0, 1).
 * Normal::compute (rand.rs:105-146): Box-Muller on xorshift128(seed_x + 2p, seed_y) and
 * xorshift128(seed_x + 2p + 1, seed_y) for the pair p = (out[2p], out[2p+1]).  The reference draws
 * both seeds from the host's thread_rng per call (rand.rs:70, 113); here the caller passes them.
 * out: dense fp32. */
int sg_rand_uniform(sg_ctx *ctx, uint32_t seed_x, uint32_t seed_y, const sg_tensor *out);
int sg_rand_normal(sg_ctx *ctx, uint32_t seed_x, uint32_t seed_y, const sg_tensor *out);

/* ---- optimizer step: optim.rs ------------------------------------------------------------------ */

/* Scalars of Adam (optim.rs:98-127).  one_minus_beta1/2 are passed, not derived: the reference's
 * beta1/beta2 are f32 fields and it forms `1.0 - self.beta` as an f32 subtraction on the host (optim.rs:152,
 * 160): 1 - 0.9f = 0.100000024, 1 - 0.999f = 0.0009999871.  The caller passes those f32 differences. */
typedef struct sg_adam_hyper {
    float lr, beta1, beta2, one_minus_beta1, one_minus_beta2, eps, weight_decay;
} sg_adam_hyper;

/* Adam::update (optim.rs:129-177) for n_tensors parameters in place, up to 32 per launch: for each i,
 * values[i], m[i], v[i] are rewritten from grads[i] by the expressions the reference builds out of map
 * operators (m' = m*beta1 + g*(1-beta1); v' = v*beta2 + pow(g,2)*(1-beta2); value' = value -
 * (m'/(1-beta1^t))*lr / (sqrt(v'/(1-beta2^t)) + eps); g = grad + value*weight_decay when that is not 0),
 * operation for operation and uncontracted: bit-identical to evaluating those operators.  step: one fp32
 * element on the device holding t (the reference keeps t as a tensor, optim.rs:165-176; it is read, not
 * advanced).  All tensors dense fp32, values[i]/grads[i]/m[i]/v[i] of equal size.  Everything is validated
 * before the first launch. */
int sg_adam_update(sg_ctx *ctx, int n_tensors, const sg_tensor *values, const sg_tensor *grads,
                   const sg_tensor *m, const sg_tensor *v, const sg_tensor *step, const sg_adam_hyper *h);

/* ---- fused row operators: compositions of ops/nn.rs ------------------------------------------ */

/* softmax over the last axis (nn.rs:42-56) of (x + addend): one pass instead of reduce(max),
 * exp(x-m) map, reduce(sum), divide map.  x: last stride 1; addend: NULL or same extents with
 * broadcast strides (the extended attention mask of bert.rs:304-314). */
int sg_softmax_lastaxis(sg_ctx *ctx, const sg_tensor *x, const sg_tensor *addend,
                        const sg_tensor *out);
/* softmax_cross_entropy (nn.rs:70-82): logits [B,C] f32, labels [B,1] uint/int, loss [B]. */
int sg_softmax_cross_entropy(sg_ctx *ctx, const sg_tensor *logits, const sg_tensor *labels,
                             const sg_tensor *loss);
/* layer_norm over the last axis (nn.rs:84-100): (x-E[x]) / sqrt(E[x^2]-E[x]^2+eps) * gamma + beta.
 * gamma, beta: numel 1 (the reference's LayerNorm holds [1] scalars, layers.rs:563-564) or numel C. */
int sg_layer_norm_lastaxis(sg_ctx *ctx, const sg_tensor *x, const sg_tensor *gamma,
                           const sg_tensor *beta, float eps, const sg_tensor *out);

/* ---- fused attention: the operator chain of MultiHeadAttention::pass (bert.rs:262-271) --------- */

/* out = softmax_lastaxis(scale * (q . k^T) + addend) . v, i.e. matmul_batched (gemm.rs:53-104), the
 * division by sqrt(head size) and the mask addition (bert.rs:264-268), Softmax::pass on axis 3
 * (layers.rs:266-273, nn.rs:42-56) and the second matmul_batched, without materialising the
 * [Lq,Lk] scores.  q, out: [.., Lq, D]; k, v: [.., Lk, D]; rank 2..4, leading axes are batch axes
 * with arbitrary strides (so the separate_heads views of bert.rs:282-291 and the merged-heads
 * output layout of bert.rs:293-302 need no copies); unit stride on D; D = 32 or 64.
 * addend: NULL or [.., Lq, Lk] holding one value per key (stride 0 over Lq, stride 1 over Lk, batch
 * strides may be 0): the extended mask of bert.rs:304-314.  The softmax shift is max(0, row max)
 * as in the reference (reduce.rs:282), so a fully masked row gives the reference's 0/0. */
int sg_attention(sg_ctx *ctx, const sg_tensor *q, const sg_tensor *k, const sg_tensor *v,
                 const sg_tensor *addend, float scale, const sg_tensor *out);

/* ---- replay of a recorded launch sequence --------------------------------------------------- */

/* Counterpart of replaying a compiled Program (Program::exec, session.rs:208-468) without the host
 * loop: every launch issued on the context between sg_graph_begin and sg_graph_end is recorded into
 * a HIP graph instead of being executed; sg_graph_launch replays all of them, on the same buffers,
 * with one submission.  Calls that wait for the device (sg_memcpy_h2d, sg_memcpy_d2h, sg_sync) are
 * refused inside a capture.  Workspaces the library allocates for captured kernels (split-K partial
 * products) stay allocated until sg_graph_destroy.  The expression kernels of sg_map must have
 * been built before the capture (run the sequence once first). */
typedef struct sg_graph sg_graph;
int sg_graph_begin(sg_ctx *ctx);
int sg_graph_end(sg_ctx *ctx, sg_graph **out);
int sg_graph_launch(sg_ctx *ctx, sg_graph *graph);
int sg_graph_destroy(sg_ctx *ctx, sg_graph *graph);

#ifdef __cplusplus
}
#endif
#endif /* SAGE_HIP_H */
