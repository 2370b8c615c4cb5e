// Fused elementwise maps: expression-specialised gfx950 kernels built at run time.
//
// The reference turns every (fused) map into OpenCL C text with the operand strides baked in and
// builds it on first use, caching by source text (map.rs:369-410, session/context.rs:62-83).  This
// file keeps that contract — one kernel per distinct expression, cached by source text — but the
// kernel it writes is shaped for CDNA4:
//   * the output index space is collapsed on the host (adjacent axes that every operand walks
//     contiguously, or broadcasts together, become one axis), so the common cases are 1-3 axes;
//   * each lane handles 4 consecutive output elements: operands whose innermost stride is 1 are
//     read with one 16-byte load, operands broadcast along the innermost axis with one 4-byte load;
//   * operands whose strides equal the output's need no index arithmetic at all ("direct", the
//     same test translate_id makes, core.rs:133-136); the others get their index from a
//     mixed-radix decomposition with magic-number division instead of the reference's per-element
//     div/mul/sub loop (core.rs:162-167);
//   * extents and strides are kernel arguments, so one build serves every shape of that class.
// Arithmetic is compiled with fp contraction off: +,-,*,/ and sqrt are then correctly rounded
// single operations and agree bit for bit with a CPU evaluation of the same expression.
#include <hip/hiprtc.h>

#include <cstring>
#include <sstream>

#include "common.h"

#include <cstdlib>

namespace {

const char *ctype(int dt) { return dt == SG_FLOAT ? "float" : dt == SG_INT ? "int" : "uint"; }

struct Gen {
    const sg_expr *prog;
    int n_prog;
    const sg_tensor *in;
    int n_in;
    int pos = 0;
    std::string err;
    int err_code = SG_OK;

    void fail(int code, const std::string &m) {
        if (err_code == SG_OK) {
            err_code = code;
            err = m;
        }
    }

    // Emits C++ text for the sub-expression at `pos` and returns the dtype the reference assigns
    // to that node when it builds the graph (map.rs:464-470, 491-501, 869-870).
    int emit(std::string &out) {
        if (pos >= n_prog) {
            fail(SG_ERR_ARG, "expression ends early");
            return SG_FLOAT;
        }
        const sg_expr e = prog[pos++];
        switch (e.kind) {
        case SG_EXPR_INPUT: {
            if (e.op < 0 || e.op >= n_in) {
                fail(SG_ERR_ARG, "input index out of range");
                return SG_FLOAT;
            }
            out += "x" + std::to_string(e.op);
            return in[e.op].dtype;
        }
        case SG_EXPR_LITERAL: {
            char buf[64];
            if (e.dtype == SG_FLOAT) snprintf(buf, sizeof buf, "__uint_as_float(0x%08xu)", e.bits);
            else if (e.dtype == SG_INT) snprintf(buf, sizeof buf, "((int)0x%08xu)", e.bits);
            else if (e.dtype == SG_UINT) snprintf(buf, sizeof buf, "0x%08xu", e.bits);
            else {
                fail(SG_ERR_DTYPE, "literal dtype must be float, int or uint");
                return SG_FLOAT;
            }
            out += buf;
            return e.dtype;
        }
        case SG_EXPR_UNARY: {
            std::string a;
            int dt = emit(a);
            static const char *fn[SG_U__COUNT] = {
                nullptr, "sg_abs", nullptr, nullptr, "logf", "expf", "sqrtf", "sg_square", "erff", "sg_sign",
                "ceilf", "floorf", "roundf", "sinf", "sinhf", "cosf", "coshf", "tanf", "tanhf",
                "asinf", "asinhf", "acosf", "acoshf", "atanf", "atanhf", nullptr, nullptr, nullptr};
            switch (e.op) {
            case SG_U_COPY: out += "(" + a + ")"; return dt;
            case SG_U_NEG: out += "(-" + a + ")"; return dt;
            case SG_U_RECIP: out += "(1/" + a + ")"; return SG_FLOAT;
            case SG_U_NOT: out += "(!" + a + ")"; return SG_UINT;
            case SG_U_CAST_INT: out += "((int)" + a + ")"; return SG_INT;
            case SG_U_CAST_FLOAT: out += "((float)" + a + ")"; return SG_FLOAT;
            default:
                if (e.op < 0 || e.op >= SG_U__COUNT || !fn[e.op]) {
                    fail(SG_ERR_ARG, "unknown unary op");
                    return SG_FLOAT;
                }
                out += std::string(fn[e.op]) + "(" + a + ")";
                return (e.op == SG_U_ABS || e.op == SG_U_SIGN) ? dt : SG_FLOAT;
            }
        }
        case SG_EXPR_BINARY: {
            std::string a, b;
            int da = emit(a), db = emit(b);
            if (da != db) fail(SG_ERR_DTYPE, "binary map operands differ in dtype (map.rs:489)");
            static const char *infix[SG_B__COUNT] = {"+", "-", "/", "*", nullptr, nullptr, nullptr, nullptr,
                                                     "&&", "||", "==", "!=", ">", ">=", "<", "<="};
            if (e.op < 0 || e.op >= SG_B__COUNT) {
                fail(SG_ERR_ARG, "unknown binary op");
                return SG_FLOAT;
            }
            if (e.op == SG_B_MOD) {
                fail(SG_ERR_ARG, "mod: the reference emits mod(a, b), which its kernel language does not define "
                                 "(map.rs:275); no kernel can be built for it");
                return SG_FLOAT;
            }
            if (infix[e.op]) out += "(" + a + " " + infix[e.op] + " " + b + ")";
            else out += std::string(e.op == SG_B_POW ? "powf" : e.op == SG_B_MIN ? "sg_min" : "sg_max") + "(" + a + ", " + b + ")";
            return e.op >= SG_B_AND ? SG_UINT : da;
        }
        case SG_EXPR_TERNARY: {
            std::string c, a, b;
            int dc = emit(c), da = emit(a), db = emit(b);
            if (e.op != SG_T_COND) fail(SG_ERR_ARG, "unknown ternary op");
            if (dc != SG_UINT) fail(SG_ERR_DTYPE, "cond: condition must be uint (map.rs:870)");
            if (da != db) fail(SG_ERR_DTYPE, "cond: branches differ in dtype (map.rs:869)");
            out += "(" + c + " ? " + a + " : " + b + ")";
            return da;
        }
        default: fail(SG_ERR_ARG, "unknown expression element"); return SG_FLOAT;
        }
    }
};

const char *kPrelude = R"SRC(
typedef float sg_float4 __attribute__((ext_vector_type(4)));
typedef int sg_int4 __attribute__((ext_vector_type(4)));
typedef unsigned int sg_uint4 __attribute__((ext_vector_type(4)));
typedef unsigned int uint;
__device__ __forceinline__ uint sg_div(uint n, uint magic, uint shift) { return (__umulhi(n, magic) + n) >> shift; }
__device__ __forceinline__ float sg_sign(float x) { return x != x ? 0.0f : (x > 0.0f ? 1.0f : (x < 0.0f ? -1.0f : x)); }
__device__ __forceinline__ float sg_sign(int x) { return sg_sign((float)x); }
__device__ __forceinline__ float sg_sign(uint x) { return sg_sign((float)x); }
__device__ __forceinline__ float sg_abs(float x) { return fabsf(x); }
__device__ __forceinline__ float sg_abs(int x) { return fabsf((float)x); }
__device__ __forceinline__ float sg_abs(uint x) { return fabsf((float)x); }
__device__ __forceinline__ float sg_square(float x) { return x * x; }
template <class A, class B> __device__ __forceinline__ auto sg_min(A a, B b) -> decltype(a + b) { decltype(a + b) x = a, y = b; return y < x ? y : x; }
template <class A, class B> __device__ __forceinline__ auto sg_max(A a, B b) -> decltype(a + b) { decltype(a + b) x = a, y = b; return x < y ? y : x; }
)SRC";

struct MapPlan {
    int ndim = 1;
    int vec = 1;
    bool stream = false;  // operands too large to be reused from cache: non-temporal loads and stores
    uint32_t ext[SG_MAX_RANK];
    uint32_t stride[SG_MAX_MAP_INPUTS][SG_MAX_RANK];
    bool direct[SG_MAX_MAP_INPUTS];
    char inner[SG_MAX_MAP_INPUTS];  // 'V' unit inner stride, 'B' broadcast along inner axis, 'S' other
    bool need_coords = false;
};

// Collapse the output index space: drop extent-1 axes, merge axis i into i+1 when every operand
// satisfies stride[i] == stride[i+1]*extent[i+1] (true for dense walks and for joint broadcasts).
void plan_map(const sg_tensor *in, int n_in, const sg_tensor *out, MapPlan &pl) {
    int64_t ext[SG_MAX_RANK];
    int64_t st[SG_MAX_MAP_INPUTS][SG_MAX_RANK];
    int nd = 0;
    for (int a = 0; a < out->rank; ++a) {
        if (out->extents[a] == 1) continue;
        ext[nd] = out->extents[a];
        for (int k = 0; k < n_in; ++k) st[k][nd] = in[k].strides[a];
        ++nd;
    }
    if (nd == 0) {
        ext[0] = 1;
        for (int k = 0; k < n_in; ++k) st[k][0] = 0;
        nd = 1;
    }
    int w = 0;  // write cursor: axes [0..w] are final so far
    for (int a = 1; a < nd; ++a) {
        bool merge = true;
        for (int k = 0; k < n_in && merge; ++k) merge = st[k][w] == st[k][a] * ext[a];
        if (merge) {
            ext[w] *= ext[a];
            for (int k = 0; k < n_in; ++k) st[k][w] = st[k][a];
        } else {
            ++w;
            ext[w] = ext[a];
            for (int k = 0; k < n_in; ++k) st[k][w] = st[k][a];
        }
    }
    nd = w + 1;
    pl.ndim = nd;
    int64_t ds[SG_MAX_RANK];
    sg_default_strides(ext, nd, ds);
    pl.need_coords = false;
    bool vec_ok = ext[nd - 1] % 4 == 0 && out->offset % 4 == 0 && ((uintptr_t)out->base % 16 == 0);
    for (int k = 0; k < n_in; ++k) {
        bool direct = true;
        for (int a = 0; a < nd; ++a) direct = direct && st[k][a] == ds[a];
        pl.direct[k] = direct;
        if (!direct) pl.need_coords = true;
        int64_t is = st[k][nd - 1];
        pl.inner[k] = is == 1 ? 'V' : is == 0 ? 'B' : 'S';
        if (pl.inner[k] == 'S') vec_ok = false;
        if (pl.inner[k] == 'V') {
            if (in[k].offset % 4 != 0 || (uintptr_t)in[k].base % 16 != 0) vec_ok = false;
            for (int a = 0; a < nd - 1; ++a)
                if (st[k][a] % 4 != 0) vec_ok = false;
        }
    }
    pl.vec = vec_ok ? 4 : 1;
    int64_t bytes = sg_numel(out) * 4;
    for (int k = 0; k < n_in; ++k) {
        int64_t distinct = 1;
        for (int a = 0; a < in[k].rank; ++a) distinct *= in[k].strides[a] != 0 ? in[k].extents[a] : 1;
        bytes += distinct * 4;
    }
    pl.stream = pl.vec == 4 && sg_streaming(bytes);
    for (int a = 0; a < nd; ++a) {
        pl.ext[a] = (uint32_t)ext[a];
        for (int k = 0; k < n_in; ++k) pl.stride[k][a] = (uint32_t)st[k][a];
    }
}

std::string gen_source(const std::string &expr, const sg_tensor *in, int n_in, int out_dt, const MapPlan &pl) {
    std::ostringstream s;
    const int nd = pl.ndim, V = pl.vec, K = n_in > 0 ? n_in : 1;
    s << kPrelude;
    s << "#define ND " << nd << "\n#define NK " << K << "\n";
    s << "struct MapParams { uint total; uint yoff; uint ext[ND]; uint magic[ND]; uint shift[ND]; uint off[NK]; uint stride[NK][ND]; };\n";
    // the expression as a function of one element of every operand
    s << "__device__ __forceinline__ " << ctype(out_dt) << " sg_expr_fn(";
    for (int k = 0; k < n_in; ++k) s << (k ? ", " : "") << ctype(in[k].dtype) << " x" << k;
    s << ") { return (" << ctype(out_dt) << ")(" << expr << "); }\n";
    s << "extern \"C\" __global__ void __launch_bounds__(256) sg_map(";
    for (int k = 0; k < n_in; ++k) s << "const " << ctype(in[k].dtype) << " *__restrict__ b" << k << ", ";
    s << ctype(out_dt) << " *__restrict__ yb, const MapParams p) {\n";
    // one 16-byte vector (or one element) per thread: measured against 2, 4 and 8 vectors per thread and
    // against grid-stride loops on 64 MB..512 MB copies and fused maps, this plain grid sustains the most
    s << "  const uint gid = blockIdx.x * 256u + threadIdx.x;\n  if (gid < p.total) {\n";
    if (pl.need_coords) {
        // coordinates in units of V elements along the innermost axis
        s << "  uint rem = gid, q;\n";
        for (int a = nd - 1; a >= 1; --a) {
            s << "  q = sg_div(rem, p.magic[" << a << "], p.shift[" << a << "]); uint c" << a << " = rem - q * p.ext[" << a << "]; rem = q;\n";
        }
        s << "  uint c0 = rem;\n";
    }
    for (int k = 0; k < n_in; ++k) {
        s << "  uint i" << k << " = p.off[" << k << "]";
        if (pl.direct[k]) {
            s << " + gid * " << V << "u";
        } else {
            for (int a = 0; a < nd; ++a) {
                if (a == nd - 1 && pl.inner[k] == 'B') continue;
                s << " + c" << a << " * p.stride[" << k << "][" << a << "]";
                if (a == nd - 1 && V > 1) s << " * " << V << "u";
            }
        }
        s << ";\n";
    }
    const char *odt = ctype(out_dt);
    if (V == 1) {
        s << "  yb[p.yoff + gid] = sg_expr_fn(";
        for (int k = 0; k < n_in; ++k) s << (k ? ", " : "") << "b" << k << "[i" << k << "]";
        s << ");\n";
    } else {
        for (int k = 0; k < n_in; ++k) {
            const char *t = ctype(in[k].dtype);
            if (pl.inner[k] == 'V')
                s << "  const sg_" << t << "4 v" << k << " = " << (pl.stream ? "__builtin_nontemporal_load(" : "*(") << "reinterpret_cast<const sg_" << t << "4 *>(b" << k << " + i" << k << "));\n";
            else
                s << "  const " << t << " s" << k << " = b" << k << "[i" << k << "];\n";
        }
        s << "  sg_" << odt << "4 r;\n";
        const char *lane[4] = {"x", "y", "z", "w"};
        for (int j = 0; j < 4; ++j) {
            s << "  r." << lane[j] << " = sg_expr_fn(";
            for (int k = 0; k < n_in; ++k) {
                s << (k ? ", " : "");
                if (pl.inner[k] == 'V') s << "v" << k << "." << lane[j];
                else s << "s" << k;
            }
            s << ");\n";
        }
        if (pl.stream) s << "  __builtin_nontemporal_store(r, reinterpret_cast<sg_" << odt << "4 *>(yb + p.yoff + gid * 4u));\n";
        else s << "  *reinterpret_cast<sg_" << odt << "4 *>(yb + p.yoff + gid * 4u) = r;\n";
    }
    s << "  }\n}\n";
    return s.str();
}

// source text -> gfx950 code object
bool compile_source(const std::string &src, std::vector<char> &code, std::string &log) {
    hiprtcProgram prog;
    if (hiprtcCreateProgram(&prog, src.c_str(), "sg_map.hip", 0, nullptr, nullptr) != HIPRTC_SUCCESS) {
        log = "hiprtcCreateProgram failed";
        return false;
    }
    // packed fp32 instructions are switched off, as for the ahead-of-time kernels
    const char *opts[] = {"--offload-arch=gfx950", "-O3", "-ffp-contract=off",
                          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
    hiprtcResult r = hiprtcCompileProgram(prog, (int)(sizeof opts / sizeof opts[0]), opts);
    if (r != HIPRTC_SUCCESS) {
        size_t n = 0;
        hiprtcGetProgramLogSize(prog, &n);
        log.assign(n, '\0');
        if (n) hiprtcGetProgramLog(prog, &log[0]);
        log = std::string(hiprtcGetErrorString(r)) + "\n" + log;
        hiprtcDestroyProgram(&prog);
        return false;
    }
    size_t csz = 0;
    hiprtcGetCodeSize(prog, &csz);
    code.resize(csz);
    hiprtcGetCode(prog, code.data());
    hiprtcDestroyProgram(&prog);
    return true;
}

int build_kernel(sg_ctx *ctx, const std::string &src, sg_jit_kernel *out) {
    std::vector<char> code;
    std::string log;
    if (!compile_source(src, code, log)) return sg_fail(ctx, SG_ERR_DEVICE, "map kernel build failed: %s", log.c_str());
    SG_HIP(ctx, hipModuleLoadData(&out->module, code.data()));
    SG_HIP(ctx, hipModuleGetFunction(&out->fn, out->module, "sg_map"));
    return SG_OK;
}

}  // namespace

extern "C" int sg_map_compile_only(const char *source, char *log_buf, uint64_t log_cap) {
    if (!source) return SG_ERR_ARG;
    std::vector<char> code;
    std::string log;
    const bool ok = compile_source(source, code, log);
    if (log_buf && log_cap) {
        size_t n = log.size() < log_cap - 1 ? log.size() : log_cap - 1;
        memcpy(log_buf, log.data(), n);
        log_buf[n] = 0;
    }
    return ok ? SG_OK : SG_ERR_DEVICE;
}

// Argument checks shared by sg_map and sg_map_source (no text is generated here).
static int map_check(sg_ctx *ctx, const sg_expr *prog, int n_prog, const sg_tensor *in, int n_in, const sg_tensor *out, bool need_ptrs) {
    if (!prog || n_prog <= 0 || n_prog > SG_MAX_EXPR) return sg_fail(ctx, SG_ERR_ARG, "sg_map: bad program length %d", n_prog);
    if (n_in < 0 || n_in > SG_MAX_MAP_INPUTS) return sg_fail(ctx, SG_ERR_ARG, "sg_map: %d inputs (max %d)", n_in, SG_MAX_MAP_INPUTS);
    if (n_in && !in) return sg_fail(ctx, SG_ERR_ARG, "sg_map: null inputs");
    if (!out) return sg_fail(ctx, SG_ERR_ARG, "sg_map: null output");
    sg_tensor tmp;
    for (int k = 0; k <= n_in; ++k) {
        const sg_tensor *t = k < n_in ? &in[k] : out;
        if (!need_ptrs && t && !t->base) {
            tmp = *t;
            tmp.base = (void *)16;
            t = &tmp;
        }
        int rc = sg_validate_tensor(ctx, t, k < n_in ? "sg_map input" : "sg_map output");
        if (rc != SG_OK) return rc;
    }
    if (!sg_is_dense(out)) return sg_fail(ctx, SG_ERR_SHAPE, "sg_map: output must be dense row-major");
    for (int k = 0; k < n_in; ++k) {
        if (in[k].rank != out->rank) return sg_fail(ctx, SG_ERR_SHAPE, "sg_map: input %d rank %d != output rank %d", k, in[k].rank, out->rank);
        for (int a = 0; a < out->rank; ++a)
            if (in[k].extents[a] != out->extents[a])
                return sg_fail(ctx, SG_ERR_SHAPE, "sg_map: input %d extent[%d] = %lld, output has %lld (ops.rs:174)", k, a,
                               (long long)in[k].extents[a], (long long)out->extents[a]);
    }
    return SG_OK;
}

// Expression text and result dtype (the dtype rules of map.rs:464-501 are enforced while emitting), then the kernel text.
static int map_generate(sg_ctx *ctx, const sg_expr *prog, int n_prog, const sg_tensor *in, int n_in, const sg_tensor *out,
                        const MapPlan &pl, std::string &src, int *res_dt) {
    Gen g{prog, n_prog, in, n_in};
    std::string expr;
    int dt = g.emit(expr);
    if (g.err_code == SG_OK && g.pos != n_prog) g.fail(SG_ERR_ARG, "expression has trailing elements");
    if (g.err_code != SG_OK) return sg_fail(ctx, g.err_code, "sg_map: %s", g.err.c_str());
    if (res_dt) *res_dt = dt;
    if (dt != out->dtype)
        return sg_fail(ctx, SG_ERR_DTYPE, "sg_map: expression yields dtype %d, output tensor is %d (map.rs:464-501)", dt, out->dtype);
    src = gen_source(expr, in, n_in, out->dtype, pl);
    return SG_OK;
}

static int map_prepare(sg_ctx *ctx, const sg_expr *prog, int n_prog, const sg_tensor *in, int n_in,
                       const sg_tensor *out, bool need_ptrs, MapPlan &pl, std::string &src, int *res_dt) {
    int rc = map_check(ctx, prog, n_prog, in, n_in, out, need_ptrs);
    if (rc != SG_OK) return rc;
    plan_map(in, n_in, out, pl);
    return map_generate(ctx, prog, n_prog, in, n_in, out, pl, src, res_dt);
}

// Everything the generated text depends on, packed into a few dozen bytes: the expression program, the operand
// dtypes and, per operand, the layout class the plan assigned (extents and strides themselves are kernel arguments).
static void map_signature(const sg_expr *prog, int n_prog, const sg_tensor *in, int n_in, const MapPlan &pl, std::string &key) {
    key.clear();
    key.reserve(16 * (size_t)n_prog + 4 * (size_t)n_in + 8);
    key.append(reinterpret_cast<const char *>(prog), sizeof(sg_expr) * (size_t)n_prog);
    const char head[4] = {(char)n_in, (char)pl.ndim, (char)pl.vec, (char)((pl.stream ? 1 : 0) | (pl.need_coords ? 2 : 0))};
    key.append(head, 4);
    for (int k = 0; k < n_in; ++k) {
        const char op[3] = {(char)in[k].dtype, (char)(pl.direct[k] ? 1 : 0), pl.inner[k]};
        key.append(op, 3);
    }
}

extern "C" int sg_map_source(sg_ctx *ctx, const sg_expr *prog, int n_prog, const sg_tensor *in, int n_in,
                             const sg_tensor *out, char *buf, uint64_t cap, int32_t *result_dtype) {
    MapPlan pl;
    std::string src;
    int dt = 0;
    int rc = map_prepare(ctx, prog, n_prog, in, n_in, out, false, pl, src, &dt);
    if (result_dtype) *result_dtype = dt;
    if (rc != SG_OK) return rc;
    if (buf && cap) {
        size_t n = src.size() < cap - 1 ? src.size() : cap - 1;
        memcpy(buf, src.data(), n);
        buf[n] = 0;
    }
    return SG_OK;
}

extern "C" int sg_map(sg_ctx *ctx, const sg_expr *prog, int n_prog, const sg_tensor *in, int n_in,
                      const sg_tensor *out) {
    if (!ctx) return SG_ERR_ARG;
    MapPlan pl;
    int rc = map_check(ctx, prog, n_prog, in, n_in, out, true);
    if (rc != SG_OK) return rc;
    plan_map(in, n_in, out, pl);

    // A repeat call of an operator finds its kernel by signature; only a new signature generates the kernel text,
    // and only a new text is built (two signatures may give the same text: the text never mentions literals' provenance).
    std::string key;
    map_signature(prog, n_prog, in, n_in, pl, key);
    auto hit = ctx->map_by_signature.find(key);
    if (hit == ctx->map_by_signature.end()) {
        std::string src;
        int dt = 0;
        rc = map_generate(ctx, prog, n_prog, in, n_in, out, pl, src, &dt);
        if (rc != SG_OK) return rc;
        auto it = ctx->jit.find(src);
        if (it == ctx->jit.end()) {
            sg_jit_kernel k{};
            rc = build_kernel(ctx, src, &k);
            if (rc != SG_OK) return rc;
            it = ctx->jit.emplace(src, k).first;
        }
        hit = ctx->map_by_signature.emplace(key, sg_map_entry{it->second.fn, dt}).first;
    } else if (hit->second.result_dtype != out->dtype) {
        return sg_fail(ctx, SG_ERR_DTYPE, "sg_map: expression yields dtype %d, output tensor is %d (map.rs:464-501)", hit->second.result_dtype, out->dtype);
    }
    const hipFunction_t fn = hit->second.fn;

    // kernel parameter block: layout must match `struct MapParams` in the generated source
    const int nd = pl.ndim, K = n_in > 0 ? n_in : 1;
    std::vector<uint32_t> params(2 + 3 * nd + K + K * nd, 0);
    const int64_t total = sg_numel(out) / pl.vec;
    params[0] = (uint32_t)total;
    params[1] = (uint32_t)out->offset;
    uint32_t *ext = &params[2], *magic = ext + nd, *shift = magic + nd, *off = shift + nd, *stride = off + K;
    for (int a = 0; a < nd; ++a) {
        uint32_t e = pl.ext[a];
        if (a == nd - 1) e /= pl.vec;
        ext[a] = e;
        sg_fastdiv f = sg_make_fastdiv(e);
        magic[a] = f.magic;
        shift[a] = f.shift;
    }
    for (int k = 0; k < n_in; ++k) {
        off[k] = (uint32_t)in[k].offset;
        for (int a = 0; a < nd; ++a) stride[k * nd + a] = pl.stride[k][a];
    }
    std::vector<void *> args;
    std::vector<const void *> ptrs(n_in + 1);
    for (int k = 0; k < n_in; ++k) {
        ptrs[k] = in[k].base;
        args.push_back(&ptrs[k]);
    }
    ptrs[n_in] = out->base;
    args.push_back(&ptrs[n_in]);
    args.push_back(params.data());
    const unsigned grid = (unsigned)((total + 255) / 256);
    SG_HIP(ctx, hipModuleLaunchKernel(fn, grid, 1, 1, 256, 1, 1, 0, ctx->stream, args.data(), nullptr));
    return SG_OK;
}
