/*
 * sage_oracle.c — CPU restatement of the reference's device kernels.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker the HIP path is compared against.  Nothing in the product
 * (sage_amd/, include/) may call, link or load it; only tests/, the smoke check and the
 * cpu_baseline leg of the benchmark do.
 *
 * Each function restates one kernel the reference generates as OpenCL C text, with the
 * reference's work decomposition (one "work-item" per output element unless noted) and its
 * arithmetic order, citing the reference file:line it follows.  Work-items are spread over host
 * threads with OpenMP (schedule(static)); inside a work-item the order of operations is the
 * reference's, so results do not depend on the thread count.
 *
 * What pins these restatements (see tests/test_oracle_*.py):
 *   - every tensor literal the reference's own unit tests hold (tests/golden/reference_literals.json)
 *   - closed forms in float64 (numpy/scipy) for maps, reductions, GEMM, im2col (torch unfold);
 *     for col2im the adjoint identity <im2col(x), c> = <x, col2im(c)>
 *   - brute-force nested-loop index checks for translate_id / gather / scatter / slice windows and for the
 *     batched product's four transpose modes;
 *   - hand-worked known answers for the integer step and the scaling of the random fills, float64 math for
 *     their Box-Muller transform.
 * Parity unpinned at ULP level: the reference evaluates exp/log/erf/pow/... and decides fma
 * contraction inside its vendor OpenCL driver, which is not part of the reference tree; these
 * restatements use the C library's float functions with contraction off.  The reference's own
 * tests pin those only to 1e-3 absolute.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "../include/sage_hip.h" /* PODs and enums only: sg_tensor, sg_expr, op codes */

#define OR_OK 0
#define OR_ERR 1

static int64_t numel(const sg_tensor *t) {
    int64_t n = 1;
    for (int i = 0; i < t->rank; ++i) n *= t->extents[i];
    return n;
}

/* Shape::default_strides (shape.rs:45-54). */
static void default_strides(const int64_t *ext, int rank, int64_t *out) {
    int64_t size = 1;
    for (int i = 0; i < rank; ++i) size *= ext[i];
    for (int i = 0; i < rank; ++i) {
        size /= ext[i] ? ext[i] : 1;
        out[i] = size;
    }
}

/* translate_id (core.rs:113-175): "direct" when the operand's strides equal the reference strides,
 * else mixed-radix decomposition of the reference id and a dot product with the operand strides.
 * The generated kernel uses 32-bit unsigned arithmetic; we keep that. */
typedef struct {
    int direct;
    int rank;
    uint32_t offset;
    uint32_t r_strides[SG_MAX_RANK];
    uint32_t t_strides[SG_MAX_RANK];
} xlate;

static void xlate_init(xlate *x, const int64_t *r_strides, int rank, const int64_t *t_strides,
                       int64_t offset) {
    x->rank = rank;
    x->offset = (uint32_t)offset;
    x->direct = 1;
    for (int i = 0; i < rank; ++i) {
        x->r_strides[i] = (uint32_t)r_strides[i];
        x->t_strides[i] = (uint32_t)t_strides[i];
        if (r_strides[i] != t_strides[i]) x->direct = 0;
    }
}

static inline uint32_t xlate_apply(const xlate *x, uint32_t gid) {
    if (x->direct) return x->offset + gid;
    uint32_t idx = x->offset, rem = gid;
    for (int i = 0; i < x->rank; ++i) {
        uint32_t c = rem / x->r_strides[i];
        rem -= c * x->r_strides[i];
        idx += c * x->t_strides[i];
    }
    return idx;
}

/* ---------------------------------------------------------------------------------------------
 * Maps.  compile_map (map.rs:369-410) + the expression text of map.rs:224-367.  The fused
 * expression is C text evaluated with C typing: loads have the buffer's type, comparisons and
 * logic yield int, mixed int/float arithmetic promotes to float, the final store converts to the
 * output type.  We evaluate the same prefix program with a small typed stack.
 * ------------------------------------------------------------------------------------------- */
typedef enum { VF = 0, VI = 1, VU = 2 } vkind;
typedef struct {
    vkind k;
    union {
        float f;
        int32_t i;
        uint32_t u;
    } v;
} val;

static inline float as_f(val a) { return a.k == VF ? a.v.f : a.k == VI ? (float)a.v.i : (float)a.v.u; }
static inline int truthy(val a) { return a.k == VF ? a.v.f != 0.0f : a.k == VI ? a.v.i != 0 : a.v.u != 0; }
static inline val mk_f(float f) { val r; r.k = VF; r.v.f = f; return r; }
static inline val mk_i(int32_t i) { val r; r.k = VI; r.v.i = i; return r; }
static inline val mk_u(uint32_t u) { val r; r.k = VU; r.v.u = u; return r; }

static inline vkind kind_of_dtype(int dt) { return dt == SG_FLOAT ? VF : dt == SG_INT ? VI : VU; }

/* OpenCL sign(): +-1, +-0 kept, NaN -> 0. */
static inline float cl_sign(float x) {
    if (x != x) return 0.0f;
    if (x > 0.0f) return 1.0f;
    if (x < 0.0f) return -1.0f;
    return x;
}

static val eval_unary(int op, val a) {
    switch (op) {
    case SG_U_COPY: return a;
    case SG_U_ABS: /* fabs(x) */
        if (a.k == VF) return mk_f(fabsf(a.v.f));
        return mk_f(fabsf(as_f(a)));
    case SG_U_NEG: /* -x */
        if (a.k == VF) return mk_f(-a.v.f);
        if (a.k == VI) return mk_i((int32_t)(0u - (uint32_t)a.v.i));
        return mk_u(0u - a.v.u);
    case SG_U_RECIP: /* 1/x : integer division for integer x */
        if (a.k == VF) return mk_f(1.0f / a.v.f);
        if (a.k == VI) return mk_i(a.v.i == 0 ? 0 : 1 / a.v.i);
        return mk_u(a.v.u == 0 ? 0 : 1u / a.v.u);
    case SG_U_LOG: return mk_f(logf(as_f(a)));
    case SG_U_EXP: return mk_f(expf(as_f(a)));
    case SG_U_SQRT: return mk_f(sqrtf(as_f(a)));
    case SG_U_SQUARE: { /* pow(x, 2) */
        float x = as_f(a);
        return mk_f(x * x);
    }
    case SG_U_ERF: return mk_f(erff(as_f(a)));
    case SG_U_SIGN: return mk_f(cl_sign(as_f(a)));
    case SG_U_CEIL: return mk_f(ceilf(as_f(a)));
    case SG_U_FLOOR: return mk_f(floorf(as_f(a)));
    case SG_U_ROUND: return mk_f(roundf(as_f(a))); /* half away from zero, as OpenCL round */
    case SG_U_SIN: return mk_f(sinf(as_f(a)));
    case SG_U_SINH: return mk_f(sinhf(as_f(a)));
    case SG_U_COS: return mk_f(cosf(as_f(a)));
    case SG_U_COSH: return mk_f(coshf(as_f(a)));
    case SG_U_TAN: return mk_f(tanf(as_f(a)));
    case SG_U_TANH: return mk_f(tanhf(as_f(a)));
    case SG_U_ASIN: return mk_f(asinf(as_f(a)));
    case SG_U_ASINH: return mk_f(asinhf(as_f(a)));
    case SG_U_ACOS: return mk_f(acosf(as_f(a)));
    case SG_U_ACOSH: return mk_f(acoshf(as_f(a)));
    case SG_U_ATAN: return mk_f(atanf(as_f(a)));
    case SG_U_ATANH: return mk_f(atanhf(as_f(a)));
    case SG_U_NOT: return mk_i(!truthy(a)); /* !x */
    case SG_U_CAST_INT: /* (int)x */
        if (a.k == VF) return mk_i((int32_t)a.v.f);
        if (a.k == VI) return a;
        return mk_i((int32_t)a.v.u);
    case SG_U_CAST_FLOAT: return mk_f(as_f(a));
    }
    return mk_f(NAN);
}

/* usual arithmetic conversions for the three 32-bit types */
static inline vkind promote(vkind a, vkind b) {
    if (a == VF || b == VF) return VF;
    if (a == VU || b == VU) return VU;
    return VI;
}
static inline uint32_t as_u(val a) { return a.k == VU ? a.v.u : a.k == VI ? (uint32_t)a.v.i : (uint32_t)a.v.f; }

static val eval_binary(int op, val a, val b) {
    vkind k = promote(a.k, b.k);
    switch (op) {
    case SG_B_ADD:
        if (k == VF) return mk_f(as_f(a) + as_f(b));
        if (k == VU) return mk_u(as_u(a) + as_u(b));
        return mk_i((int32_t)((uint32_t)a.v.i + (uint32_t)b.v.i));
    case SG_B_SUB:
        if (k == VF) return mk_f(as_f(a) - as_f(b));
        if (k == VU) return mk_u(as_u(a) - as_u(b));
        return mk_i((int32_t)((uint32_t)a.v.i - (uint32_t)b.v.i));
    case SG_B_MUL:
        if (k == VF) return mk_f(as_f(a) * as_f(b));
        if (k == VU) return mk_u(as_u(a) * as_u(b));
        return mk_i((int32_t)((uint32_t)a.v.i * (uint32_t)b.v.i));
    case SG_B_DIV:
        if (k == VF) return mk_f(as_f(a) / as_f(b));
        if (k == VU) return mk_u(as_u(b) ? as_u(a) / as_u(b) : 0);
        return mk_i(b.v.i ? (b.v.i == -1 ? (int32_t)(0u - (uint32_t)a.v.i) : a.v.i / b.v.i) : 0);
    case SG_B_POW: return mk_f(powf(as_f(a), as_f(b)));
    case SG_B_MIN: /* OpenCL min(x,y) = y < x ? y : x */
        if (k == VF) { float x = as_f(a), y = as_f(b); return mk_f(y < x ? y : x); }
        if (k == VU) { uint32_t x = as_u(a), y = as_u(b); return mk_u(y < x ? y : x); }
        return mk_i(b.v.i < a.v.i ? b.v.i : a.v.i);
    case SG_B_MAX: /* OpenCL max(x,y) = x < y ? y : x */
        if (k == VF) { float x = as_f(a), y = as_f(b); return mk_f(x < y ? y : x); }
        if (k == VU) { uint32_t x = as_u(a), y = as_u(b); return mk_u(x < y ? y : x); }
        return mk_i(a.v.i < b.v.i ? b.v.i : a.v.i);
    case SG_B_AND: return mk_i(truthy(a) && truthy(b));
    case SG_B_OR: return mk_i(truthy(a) || truthy(b));
    default: break;
    }
    /* comparisons: int 0/1 */
    int r = 0;
    if (k == VF) {
        float x = as_f(a), y = as_f(b);
        switch (op) {
        case SG_B_EQ: r = x == y; break;
        case SG_B_NE: r = x != y; break;
        case SG_B_GT: r = x > y; break;
        case SG_B_GE: r = x >= y; break;
        case SG_B_LT: r = x < y; break;
        case SG_B_LE: r = x <= y; break;
        }
    } else if (k == VU) {
        uint32_t x = as_u(a), y = as_u(b);
        switch (op) {
        case SG_B_EQ: r = x == y; break;
        case SG_B_NE: r = x != y; break;
        case SG_B_GT: r = x > y; break;
        case SG_B_GE: r = x >= y; break;
        case SG_B_LT: r = x < y; break;
        case SG_B_LE: r = x <= y; break;
        }
    } else {
        int32_t x = a.v.i, y = b.v.i;
        switch (op) {
        case SG_B_EQ: r = x == y; break;
        case SG_B_NE: r = x != y; break;
        case SG_B_GT: r = x > y; break;
        case SG_B_GE: r = x >= y; break;
        case SG_B_LT: r = x < y; break;
        case SG_B_LE: r = x <= y; break;
        }
    }
    return mk_i(r);
}

/* Evaluate the prefix program the way VariadicMapOperator::map_fn walks it (map.rs:303-367):
 * scan from the end, push operands, apply an operator to the topmost values with the top being
 * its first operand. */
static val eval_prog(const sg_expr *prog, int n_prog, const val *inputs) {
    val stack[SG_MAX_EXPR];
    int sp = 0;
    for (int p = n_prog - 1; p >= 0; --p) {
        const sg_expr *e = &prog[p];
        switch (e->kind) {
        case SG_EXPR_INPUT: stack[sp++] = inputs[e->op]; break;
        case SG_EXPR_LITERAL: {
            val l;
            l.k = kind_of_dtype(e->dtype);
            l.v.u = e->bits;
            stack[sp++] = l;
            break;
        }
        case SG_EXPR_UNARY: stack[sp - 1] = eval_unary(e->op, stack[sp - 1]); break;
        case SG_EXPR_BINARY: {
            val a = stack[sp - 1], b = stack[sp - 2];
            sp -= 1;
            stack[sp - 1] = eval_binary(e->op, a, b);
            break;
        }
        case SG_EXPR_TERNARY: { /* c ? a : b   (map.rs:299) */
            val c = stack[sp - 1], a = stack[sp - 2], b = stack[sp - 3];
            sp -= 2;
            val r = truthy(c) ? a : b;
            if (a.k != b.k) { /* C: both arms converted to the common type */
                vkind k = promote(a.k, b.k);
                if (k == VF) r = mk_f(as_f(r));
                else if (k == VU) r = mk_u(as_u(r));
            }
            stack[sp - 1] = r;
            break;
        }
        }
    }
    return stack[0];
}

int or_map(const sg_expr *prog, int n_prog, const sg_tensor *in, int n_in, const sg_tensor *out) {
    if (n_prog <= 0 || n_prog > SG_MAX_EXPR || n_in > SG_MAX_MAP_INPUTS) return OR_ERR;
    for (int p = 0; p < n_prog; ++p)
        if (prog[p].kind == SG_EXPR_BINARY && prog[p].op == SG_B_MOD) return OR_ERR; /* map.rs:275 */
    int64_t n = numel(out);
    int64_t rs[SG_MAX_RANK];
    default_strides(out->extents, out->rank, rs);
    xlate xl[SG_MAX_MAP_INPUTS];
    for (int i = 0; i < n_in; ++i) xlate_init(&xl[i], rs, out->rank, in[i].strides, in[i].offset);
    vkind ok = kind_of_dtype(out->dtype);
    uint32_t *y = (uint32_t *)out->base + out->offset;
#pragma omp parallel for schedule(static)
    for (int64_t gid = 0; gid < n; ++gid) {
        val inputs[SG_MAX_MAP_INPUTS];
        for (int i = 0; i < n_in; ++i) {
            uint32_t idx = xlate_apply(&xl[i], (uint32_t)gid);
            inputs[i].k = kind_of_dtype(in[i].dtype);
            inputs[i].v.u = ((const uint32_t *)in[i].base)[idx];
        }
        val r = eval_prog(prog, n_prog, inputs);
        /* y[gid] = expr;  -> conversion to the output element type */
        if (ok == VF) { float f = as_f(r); memcpy(&y[gid], &f, 4); }
        else if (ok == VI) { int32_t i = r.k == VF ? (int32_t)r.v.f : (int32_t)as_u(r); memcpy(&y[gid], &i, 4); }
        else { uint32_t u = r.k == VF ? (uint32_t)r.v.f : as_u(r); y[gid] = u; }
    }
    return OR_OK;
}

/* ---------------------------------------------------------------------------------------------
 * Reductions.  ReduceOperator::compute (reduce.rs:258-325): one work-item per output element;
 * outer index via translate_id over the kept axes; nested loops over the reduced axes with the
 * FIRST listed axis innermost (reduce.rs:296-315); accumulator starts at literal 0 (reduce.rs:282)
 * unless init_mode asks for the mathematical identity.
 * ------------------------------------------------------------------------------------------- */
static void split_axes(const sg_tensor *t, const int32_t *axes, int n_axes, int64_t *in_ext,
                       int64_t *in_str, int64_t *out_ext, int64_t *out_str, int *n_out) {
    /* Shape::extract (shape.rs:113-132): inner = the listed axes in listed order, outer = the rest */
    for (int i = 0; i < n_axes; ++i) {
        in_ext[i] = t->extents[axes[i]];
        in_str[i] = t->strides[axes[i]];
    }
    int m = 0;
    for (int a = 0; a < t->rank; ++a) {
        int listed = 0;
        for (int i = 0; i < n_axes; ++i) listed |= axes[i] == a;
        if (!listed) {
            out_ext[m] = t->extents[a];
            out_str[m] = t->strides[a];
            ++m;
        }
    }
    *n_out = m;
}

int or_reduce(int op, const int32_t *axes, int n_axes, int init_mode, const sg_tensor *in,
              const sg_tensor *out) {
    int64_t ie[SG_MAX_RANK], is[SG_MAX_RANK], oe[SG_MAX_RANK], os[SG_MAX_RANK], ods[SG_MAX_RANK];
    int n_out;
    if (n_axes < 0 || n_axes > in->rank) return OR_ERR;
    split_axes(in, axes, n_axes, ie, is, oe, os, &n_out);
    default_strides(oe, n_out, ods);
    xlate xo;
    xlate_init(&xo, ods, n_out, os, in->offset);
    int64_t n = numel(out);
    int64_t inner = 1;
    for (int i = 0; i < n_axes; ++i) inner *= ie[i];
    int dt = in->dtype;
    uint32_t *y = (uint32_t *)out->base + out->offset;
    const uint32_t *x = (const uint32_t *)in->base;
#pragma omp parallel for schedule(static)
    for (int64_t gid = 0; gid < n; ++gid) {
        uint32_t outer_idx = xlate_apply(&xo, (uint32_t)gid);
        int64_t c[SG_MAX_RANK] = {0};
        if (dt == SG_FLOAT) {
            float acc = 0.0f;
            if (init_mode == SG_INIT_IDENTITY)
                acc = op == SG_R_PROD ? 1.0f : op == SG_R_MAX ? -INFINITY : op == SG_R_MIN ? INFINITY : 0.0f;
            for (int64_t it = 0; it < inner; ++it) {
                uint32_t inner_idx = 0;
                for (int i = 0; i < n_axes; ++i) inner_idx += (uint32_t)(c[i] * is[i]);
                float v;
                memcpy(&v, &x[outer_idx + inner_idx], 4);
                switch (op) {
                case SG_R_SUM: acc = acc + v; break;
                case SG_R_PROD: acc = acc * v; break;
                case SG_R_MAX: acc = acc < v ? v : acc; break; /* max(acc, val) */
                case SG_R_MIN: acc = v < acc ? v : acc; break; /* min(acc, val) */
                }
                for (int i = 0; i < n_axes; ++i) { /* axis 0 of the list is the innermost loop */
                    if (++c[i] < ie[i]) break;
                    c[i] = 0;
                }
            }
            memcpy(&y[gid], &acc, 4);
        } else {
            int is_signed = dt == SG_INT;
            int64_t acc = 0;
            if (init_mode == SG_INIT_IDENTITY)
                acc = op == SG_R_PROD ? 1
                      : op == SG_R_MAX ? (is_signed ? INT32_MIN : 0)
                      : op == SG_R_MIN ? (is_signed ? INT32_MAX : (int64_t)UINT32_MAX) : 0;
            for (int64_t it = 0; it < inner; ++it) {
                uint32_t inner_idx = 0;
                for (int i = 0; i < n_axes; ++i) inner_idx += (uint32_t)(c[i] * is[i]);
                uint32_t raw = x[outer_idx + inner_idx];
                int64_t v = is_signed ? (int64_t)(int32_t)raw : (int64_t)raw;
                switch (op) {
                case SG_R_SUM: acc = (int64_t)(uint32_t)((uint32_t)acc + (uint32_t)v); break;
                case SG_R_PROD: acc = (int64_t)(uint32_t)((uint32_t)acc * (uint32_t)v); break;
                case SG_R_MAX: acc = acc < v ? v : acc; break;
                case SG_R_MIN: acc = v < acc ? v : acc; break;
                }
                if (is_signed && (op == SG_R_SUM || op == SG_R_PROD)) acc = (int64_t)(int32_t)(uint32_t)acc;
                for (int i = 0; i < n_axes; ++i) {
                    if (++c[i] < ie[i]) break;
                    c[i] = 0;
                }
            }
            y[gid] = (uint32_t)acc;
        }
    }
    return OR_OK;
}

/* ReduceArgOperator::compute (reduce.rs:372-431): acc = x[outer], arg = 0, strict compare. */
int or_reduce_arg(int op, int axis, const sg_tensor *in, const sg_tensor *out) {
    int64_t ie[1], is[1], oe[SG_MAX_RANK], os[SG_MAX_RANK], ods[SG_MAX_RANK];
    int n_out;
    int32_t ax = axis;
    if (axis < 0 || axis >= in->rank) return OR_ERR;
    split_axes(in, &ax, 1, ie, is, oe, os, &n_out);
    default_strides(oe, n_out, ods);
    xlate xo;
    xlate_init(&xo, ods, n_out, os, in->offset);
    int64_t n = numel(out);
    int dt = in->dtype;
    const uint32_t *x = (const uint32_t *)in->base;
    uint32_t *y = (uint32_t *)out->base + out->offset;
#pragma omp parallel for schedule(static)
    for (int64_t gid = 0; gid < n; ++gid) {
        uint32_t outer_idx = xlate_apply(&xo, (uint32_t)gid);
        uint32_t arg = 0;
        if (dt == SG_FLOAT) {
            float acc;
            memcpy(&acc, &x[outer_idx], 4);
            for (int64_t i = 0; i < ie[0]; ++i) {
                float v;
                memcpy(&v, &x[outer_idx + (uint32_t)(i * is[0])], 4);
                if (op == SG_RA_MAX ? acc < v : acc > v) { arg = (uint32_t)i; acc = v; }
            }
        } else {
            int sgn = dt == SG_INT;
            int64_t acc = sgn ? (int64_t)(int32_t)x[outer_idx] : (int64_t)x[outer_idx];
            for (int64_t i = 0; i < ie[0]; ++i) {
                uint32_t raw = x[outer_idx + (uint32_t)(i * is[0])];
                int64_t v = sgn ? (int64_t)(int32_t)raw : (int64_t)raw;
                if (op == SG_RA_MAX ? acc < v : acc > v) { arg = (uint32_t)i; acc = v; }
            }
        }
        y[gid] = arg;
    }
    return OR_OK;
}

/* ---------------------------------------------------------------------------------------------
 * Indexing kernels (core.rs).
 * ------------------------------------------------------------------------------------------- */

/* Gather::compute (core.rs:655-718). */
int or_gather(int axis, const sg_tensor *x, const sg_tensor *ind, const sg_tensor *out) {
    int rank = x->rank;
    if (ind->rank != rank || axis < 0 || axis >= rank) return OR_ERR;
    int64_t sd[SG_MAX_RANK];
    default_strides(ind->extents, rank, sd);
    xlate xi;
    xlate_init(&xi, sd, rank, ind->strides, 0);
    int64_t n = numel(out);
    const uint32_t *xb = (const uint32_t *)x->base;
    const uint32_t *ib = (const uint32_t *)ind->base;
    uint32_t *y = (uint32_t *)out->base;
#pragma omp parallel for schedule(static)
    for (int64_t gid = 0; gid < n; ++gid) {
        uint32_t idx = (uint32_t)x->offset;
        uint32_t gather_idx = xlate_apply(&xi, (uint32_t)gid);
        uint32_t target = ib[gather_idx + (uint32_t)ind->offset];
        uint32_t rem = (uint32_t)gid;
        for (int i = 0; i < rank; ++i) {
            uint32_t c = rem / (uint32_t)sd[i];
            rem -= c * (uint32_t)sd[i];
            idx += (i == axis ? target : c) * (uint32_t)x->strides[i];
        }
        y[gid + out->offset] = xb[idx];
    }
    return OR_OK;
}

/* Scatter::compute (core.rs:764-833): zero-fill, then a read-modify-write per index element.  The
 * reference decomposes gid by ind's OWN strides (core.rs:770) and runs its work-items
 * concurrently without atomics; here they run one after another in gid order, which is what the
 * reference computes whenever no two work-items hit the same output element. */
int or_scatter(int axis, const sg_tensor *x, const sg_tensor *ind, const sg_tensor *out) {
    int rank = out->rank;
    if (ind->rank != rank || x->rank != rank || axis < 0 || axis >= rank) return OR_ERR;
    int64_t n_out = numel(out), n = numel(ind);
    int64_t sd_ref[SG_MAX_RANK];
    default_strides(ind->extents, rank, sd_ref);
    xlate xi;
    xlate_init(&xi, sd_ref, rank, ind->strides, 0);
    for (int i = 0; i < rank; ++i)
        if (ind->strides[i] == 0) return OR_ERR; /* division by zero in the reference kernel */
    uint32_t *y = (uint32_t *)out->base;
    memset(y + out->offset, 0, (size_t)n_out * 4);
    const uint32_t *xb = (const uint32_t *)x->base;
    const uint32_t *ib = (const uint32_t *)ind->base;
    for (int64_t gid = 0; gid < n; ++gid) {
        uint32_t idx_in = (uint32_t)x->offset, idx_out = (uint32_t)out->offset;
        uint32_t sidx = xlate_apply(&xi, (uint32_t)gid);
        uint32_t target = ib[sidx + (uint32_t)ind->offset];
        uint32_t rem = (uint32_t)gid;
        for (int i = 0; i < rank; ++i) {
            uint32_t c = rem / (uint32_t)ind->strides[i];
            rem -= c * (uint32_t)ind->strides[i];
            idx_in += c * (uint32_t)x->strides[i];
            idx_out += (i == axis ? target : c) * (uint32_t)out->strides[i];
        }
        /* y[idx_out + y_offset] += x[idx_in]; a fresh output has offset 0 (core.rs:795,816) */
        if (x->dtype == SG_FLOAT) {
            float a, b;
            memcpy(&a, &y[idx_out], 4);
            memcpy(&b, &xb[idx_in], 4);
            a += b;
            memcpy(&y[idx_out], &a, 4);
        } else {
            y[idx_out] += xb[idx_in];
        }
    }
    return OR_OK;
}

/* Unslice::compute (core.rs:553-611). */
int or_unslice(int axis, int64_t start, const sg_tensor *x, const sg_tensor *out) {
    int rank = x->rank;
    int64_t rs[SG_MAX_RANK];
    default_strides(x->extents, rank, rs);
    xlate xin, xout;
    xlate_init(&xin, rs, rank, x->strides, x->offset);
    xlate_init(&xout, rs, rank, out->strides, out->offset + start * out->strides[axis]);
    uint32_t *y = (uint32_t *)out->base;
    memset(y + out->offset, 0, (size_t)numel(out) * 4);
    const uint32_t *xb = (const uint32_t *)x->base;
    int64_t n = numel(x);
#pragma omp parallel for schedule(static)
    for (int64_t gid = 0; gid < n; ++gid) y[xlate_apply(&xout, (uint32_t)gid)] = xb[xlate_apply(&xin, (uint32_t)gid)];
    return OR_OK;
}

/* Concat::compute (core.rs:892-934). */
int or_concat(int axis, const sg_tensor *in, int n_in, const sg_tensor *out) {
    uint32_t *y = (uint32_t *)out->base;
    memset(y + out->offset, 0, (size_t)numel(out) * 4);
    int64_t at = 0;
    for (int k = 0; k < n_in; ++k) {
        const sg_tensor *v = &in[k];
        int64_t rs[SG_MAX_RANK];
        default_strides(v->extents, v->rank, rs);
        xlate xin, xout;
        xlate_init(&xin, rs, v->rank, v->strides, v->offset);
        /* y.shape().select_range(i, i+e-1, axis): offset += stride*i (shape.rs:230-237) */
        xlate_init(&xout, rs, v->rank, out->strides, out->offset + at * out->strides[axis]);
        at += v->extents[axis];
        const uint32_t *xb = (const uint32_t *)v->base;
        int64_t n = numel(v);
#pragma omp parallel for schedule(static)
        for (int64_t gid = 0; gid < n; ++gid) y[xlate_apply(&xout, (uint32_t)gid)] = xb[xlate_apply(&xin, (uint32_t)gid)];
    }
    return OR_OK;
}

/* ---------------------------------------------------------------------------------------------
 * GEMM.  Gemm::compute_direct (gemm.rs:176-250) launching XgemmDirect (matmul_direct.opencl:514-709)
 * with alpha 1, beta 0, c_transpose = 1 (row-major C).  Index conventions: A[m,k] at m*lda+k, or
 * k*lda+m when transpose_a; B[k,n] at k*ldb+n, or n*ldb+k when transpose_b; C[m,n] at m*ldc+n.
 * Each output accumulates k = 0..K-1 in order with `acc += a*b` (matmul_direct.opencl:573-597).
 * The loop nest below is m / k / n: per output element that is the same order of additions.
 * ------------------------------------------------------------------------------------------- */
static void gemm_one(int ta, int tb, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                     const float *B, int64_t ldb, float *C, int64_t ldc) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        float *c = C + m * ldc;
        for (int64_t n = 0; n < N; ++n) c[n] = 0.0f; /* fill_zero(y), gemm.rs:179 */
        for (int64_t k = 0; k < K; ++k) {
            float a = ta ? A[k * lda + m] : A[m * lda + k];
            if (!tb) {
                const float *b = B + k * ldb;
                for (int64_t n = 0; n < N; ++n) c[n] += a * b[n];
            } else {
                for (int64_t n = 0; n < N; ++n) c[n] += a * B[n * ldb + k];
            }
        }
    }
}

int or_gemm(int ta, int tb, const sg_tensor *a, const sg_tensor *b, const sg_tensor *c) {
    if (a->rank != 2 || b->rank != 2 || c->rank != 2) return OR_ERR;
    int64_t M = a->extents[ta ? 1 : 0], K = a->extents[ta ? 0 : 1];
    int64_t N = b->extents[tb ? 0 : 1], K2 = b->extents[tb ? 1 : 0];
    if (K != K2 || c->extents[0] != M || c->extents[1] != N) return OR_ERR;
    gemm_one(ta, tb, M, N, K, (const float *)a->base + a->offset, a->strides[0],
             (const float *)b->base + b->offset, b->strides[0], (float *)c->base + c->offset,
             c->strides[0]);
    return OR_OK;
}

/* GemmBatched::compute_direct (gemm.rs:338-421): batch = group id 2, matrix b at base + stride*b. */
int or_gemm_batched(int ta, int tb, const sg_tensor *a, const sg_tensor *b, const sg_tensor *c) {
    if (a->rank != 3 || b->rank != 3 || c->rank != 3) return OR_ERR;
    int64_t batch = a->extents[0];
    int64_t M = a->extents[ta ? 2 : 1], K = a->extents[ta ? 1 : 2];
    int64_t N = b->extents[tb ? 1 : 2], K2 = b->extents[tb ? 2 : 1];
    if (K != K2 || b->extents[0] != batch || c->extents[0] != batch || c->extents[1] != M || c->extents[2] != N)
        return OR_ERR;
    for (int64_t i = 0; i < batch; ++i)
        gemm_one(ta, tb, M, N, K, (const float *)a->base + a->offset + i * a->strides[0], a->strides[1],
                 (const float *)b->base + b->offset + i * b->strides[0], b->strides[1],
                 (float *)c->base + c->offset + i * c->strides[0], c->strides[1]);
    return OR_OK;
}

/* ---------------------------------------------------------------------------------------------
 * Im2col::compute (conv.rs:289-374).  Work-item = (col_y, col_x, c); batch, ker_y, ker_x are
 * looped inside it.  Pairs are {w, h}.
 * ------------------------------------------------------------------------------------------- */
int or_im2col(const sg_tensor *x, const sg_tensor *out, const int32_t ker[2], const int32_t stride[2],
              const int32_t pad[2], const int32_t dil[2]) {
    if (x->rank != 4 || out->rank != 6) return OR_ERR;
    int batch = (int)x->extents[0], img_h = (int)x->extents[1], img_w = (int)x->extents[2], chan = (int)x->extents[3];
    int col_h = (int)out->extents[1], col_w = (int)out->extents[2];
    int ker_w = ker[0], ker_h = ker[1];
    const float *img = (const float *)x->base;
    float *col = (float *)out->base;
    int img_offset = (int)x->offset, col_offset = (int)out->offset;
    int gws = col_w * col_h * chan;
#pragma omp parallel for schedule(static)
    for (int gid = 0; gid < gws; ++gid) {
        for (int n = 0; n < batch; ++n) {
            int offset_img_batch = n * img_h * img_w * chan;
            int offset_col_batch = n * col_h * col_w * ker_h * ker_w * chan;
            int c = gid % chan;
            int col_x = (gid / chan) % col_w;
            int col_y = gid / (chan * col_w);
            int img_x_base = col_x * stride[0] - pad[0];
            int img_y_base = col_y * stride[1] - pad[1];
            for (int ker_y = 0; ker_y < ker_h; ++ker_y) {
                for (int ker_x = 0; ker_x < ker_w; ++ker_x) {
                    int img_y = img_y_base + ker_y * dil[1];
                    int img_x = img_x_base + ker_x * dil[0];
                    int offset_col = offset_col_batch + (((col_y * col_w + col_x) * ker_h + ker_y) * ker_w + ker_x) * chan + col_offset;
                    float v = 0.0f;
                    if (img_x >= 0 && img_x < img_w && img_y >= 0 && img_y < img_h) {
                        int offset_img = offset_img_batch + (img_y * img_w + img_x) * chan + img_offset;
                        v = img[offset_img + c];
                    }
                    col[offset_col + c] = v;
                }
            }
        }
    }
    return OR_OK;
}

/* ---------------------------------------------------------------------------------------------
 * Col2im::compute (conv.rs:405-500).  Work-item = (img_y, img_x, c); the batch and the contributing
 * columns are looped inside it, col_x outer and col_y inner (the order of the float additions).
 * The reference tests ker_x against dilation_h and ker_y against dilation_w (conv.rs:463-465) and
 * divides by them; kept as is.  Where the two dilations differ (and the kernel has more than one tap)
 * the tap indices that come out of that lie outside [0, ker): the reference's kernel then reads
 * entries of other taps or past the end of its buffer, i.e. it defines no result; this restatement
 * refuses such a geometry (OR_ERR) instead of reading out of bounds.  Pairs are {w, h}.
 * ------------------------------------------------------------------------------------------- */
int or_col2im(const sg_tensor *x, const sg_tensor *out, const int32_t ker[2], const int32_t stride[2],
              const int32_t pad[2], const int32_t dil[2]) {
    if (x->rank != 6 || out->rank != 4) return OR_ERR;
    if (dil[0] != dil[1] && (ker[0] > 1 || ker[1] > 1)) return OR_ERR; /* undefined in the reference, see above */
    int batch = (int)x->extents[0], col_h = (int)x->extents[1], col_w = (int)x->extents[2], chan = (int)x->extents[5];
    int img_h = (int)out->extents[1], img_w = (int)out->extents[2];
    int ker_w = ker[0], ker_h = ker[1], stride_w = stride[0], stride_h = stride[1];
    int padding_w = pad[0], padding_h = pad[1], dilation_w = dil[0], dilation_h = dil[1];
    const float *col = (const float *)x->base;
    float *img = (float *)out->base;
    int col_offset = (int)x->offset, img_offset = (int)out->offset;
    int gws = img_w * img_h * chan;
#pragma omp parallel for schedule(static)
    for (int gid = 0; gid < gws; ++gid) {
        for (int n = 0; n < batch; ++n) {
            int offset_img_batch = n * img_h * img_w * chan;
            int offset_col_batch = n * col_h * col_w * ker_h * ker_w * chan;
            int c = gid % chan;
            int img_x = (gid / chan) % img_w;
            int img_y = gid / (chan * img_w);
            int img_x_pad = img_x + padding_w, img_y_pad = img_y + padding_h;
            int ker_ew = (ker_w - 1) * dilation_w + 1, ker_eh = (ker_h - 1) * dilation_h + 1;
            int col_x_start = (img_x_pad < ker_ew) ? 0 : (img_x_pad - ker_ew) / stride_w + 1;
            int col_y_start = (img_y_pad < ker_eh) ? 0 : (img_y_pad - ker_eh) / stride_h + 1;
            int col_x_end = img_x_pad / stride_w + 1 < col_w ? img_x_pad / stride_w + 1 : col_w;
            int col_y_end = img_y_pad / stride_h + 1 < col_h ? img_y_pad / stride_h + 1 : col_h;
            float val = 0.0f;
            int offset_img = (img_y * img_w + img_x) * chan + img_offset;
            for (int col_x = col_x_start; col_x < col_x_end; ++col_x) {
                for (int col_y = col_y_start; col_y < col_y_end; ++col_y) {
                    int ker_x = img_x_pad - col_x * stride_w;
                    int ker_y = img_y_pad - col_y * stride_h;
                    if (ker_x % dilation_h == 0 && ker_y % dilation_w == 0) {
                        ker_x /= dilation_h;
                        ker_y /= dilation_w;
                        int offset_col = (((col_y * col_w + col_x) * ker_h + ker_y) * ker_w + ker_x) * chan + col_offset;
                        val += col[offset_col_batch + offset_col + c];
                    }
                }
            }
            img[offset_img_batch + offset_img + c] = val;
        }
    }
    return OR_OK;
}

/* ---------------------------------------------------------------------------------------------
 * Uniform::compute / Normal::compute (rand.rs:39-49, 77-83, 120-136) for given seeds.
 *
 * The kernels are OpenCL C text built without compiler options (device.rs passes none), so an unsuffixed
 * floating literal and M_PI are DOUBLE on the fp64-capable devices the reference selects:
 *   xorshift128 returns (float)((double)rndint * 2.3283064e-10)   -- one rounding, not (float)rndint * 2^-32
 *                                                                    (the two differ by an ulp for one seed in five);
 *   theta = (float)(2 * M_PI * (double)u2);  rsq = -2 * log(u1) stays float (integer literal).
 * The integer step is pinned by hand-worked known answers and the scaling by a seed on which the two readings
 * differ (tests/test_oracle_golden.py); the Box-Muller values by float64 math.  log/cos/sin themselves are the C
 * library's here and the driver's in the reference: unpinned at ULP level like every transcendental.
 * The odd trailing element of the normal fill is the cosine branch only (the reference writes one float past
 * its buffer there).
 * ------------------------------------------------------------------------------------------- */
static float or_xorshift128(uint32_t seed_x, uint32_t seed_y) {
    const uint32_t t = seed_x ^ (seed_x << 11);
    const uint32_t rndint = seed_y ^ (seed_y >> 19) ^ (t ^ (t >> 8));
    return (float)((double)rndint * 2.3283064e-10);
}

int or_rand_uniform(uint32_t seed_x, uint32_t seed_y, const sg_tensor *out) {
    float *y = (float *)out->base + out->offset;
    int64_t n = numel(out);
    for (int64_t gid = 0; gid < n; ++gid) y[gid] = or_xorshift128(seed_x + (uint32_t)gid, seed_y + (uint32_t)gid);
    return OR_OK;
}

int or_rand_normal(uint32_t seed_x, uint32_t seed_y, const sg_tensor *out) {
    float *y = (float *)out->base + out->offset;
    int64_t n = numel(out);
    for (int64_t gid = 0; 2 * gid < n; ++gid) {
        const float u1 = or_xorshift128(seed_x + (uint32_t)gid * 2u, seed_y);
        const float u2 = or_xorshift128(seed_x + (uint32_t)gid * 2u + 1u, seed_y);
        const float rsq = -2.0f * logf(u1);
        const float theta = (float)(2.0 * 3.14159265358979323846 * (double)u2);
        y[2 * gid] = sqrtf(rsq) * cosf(theta);
        if (2 * gid + 1 < n) y[2 * gid + 1] = sqrtf(rsq) * sinf(theta);
    }
    return OR_OK;
}

int or_num_threads(void) {
#ifdef _OPENMP
    extern int omp_get_max_threads(void);
    return omp_get_max_threads();
#else
    return 1;
#endif
}
