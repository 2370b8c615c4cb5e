"""ctypes binding of include/sage_hip.h — the C ABI of the gfx950 backend.

This is the binding a maintainer of the reference would write for its own host language; nothing
here computes anything.  Loading fails loudly when the built library is missing: there is no CPU
fallback of any kind.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libsage_hip.so")

MAX_RANK = 8
MAX_MAP_INPUTS = 16
MAX_EXPR = 128
REFERENCE_CAPACITY_BYTES = 1000 * 1024 * 1024
GEMM_NOALLOC_SCRATCH_BYTES = 32 << 20

OK, ERR_OOM, ERR_DEVICE, ERR_SHAPE, ERR_DTYPE, ERR_ARG = range(6)
CHAR, SHORT, INT, LONG, UCHAR, USHORT, UINT, ULONG, FLOAT, HALF = range(10)

UNARY = ("copy abs neg recip log exp sqrt square erf sign ceil floor round sin sinh cos cosh tan tanh "
         "asin asinh acos acosh atan atanh not cast_int cast_float").split()
BINARY = "add sub div mul mod pow min max and or eq ne gt ge lt le".split()
U = {n: i for i, n in enumerate(UNARY)}
B = {n: i for i, n in enumerate(BINARY)}
EXPR_INPUT, EXPR_LITERAL, EXPR_UNARY, EXPR_BINARY, EXPR_TERNARY = range(5)
R_SUM, R_PROD, R_MAX, R_MIN = range(4)
RA_MAX, RA_MIN = 0, 1
INIT_REF_ZERO, INIT_IDENTITY = 0, 1
ACT_NONE, ACT_RELU, ACT_GELU_ERF = 0, 1, 2


class sg_tensor(C.Structure):
    _fields_ = [("base", C.c_void_p), ("dtype", C.c_int32), ("rank", C.c_int32),
                ("extents", C.c_int64 * MAX_RANK), ("strides", C.c_int64 * MAX_RANK),
                ("offset", C.c_int64)]


class sg_expr(C.Structure):
    _fields_ = [("kind", C.c_int32), ("op", C.c_int32), ("dtype", C.c_int32), ("bits", C.c_uint32)]


class sg_gemm_epilogue(C.Structure):
    _fields_ = [("alpha", C.c_float), ("act", C.c_int32), ("act_post", C.c_int32),
                ("bias", C.POINTER(sg_tensor)), ("residual", C.POINTER(sg_tensor))]


class sg_adam_hyper(C.Structure):
    _fields_ = [("lr", C.c_float), ("beta1", C.c_float), ("beta2", C.c_float), ("one_minus_beta1", C.c_float),
                ("one_minus_beta2", C.c_float), ("eps", C.c_float), ("weight_decay", C.c_float)]


_TP = C.POINTER(sg_tensor)
_CTX = C.c_void_p
_I32P = C.POINTER(C.c_int32)
_U64P = C.POINTER(C.c_uint64)

# name -> (restype, argtypes): every symbol include/sage_hip.h declares
PROTOTYPES = {
    "sg_ctx_create": (C.c_int, [C.c_int, C.c_uint64, C.POINTER(_CTX)]),
    "sg_ctx_create_pooled": (C.c_int, [C.c_int, C.c_uint64, C.c_int, C.c_int, C.POINTER(_CTX)]),
    "sg_ctx_destroy": (C.c_int, [_CTX]),
    "sg_alloc": (C.c_int, [_CTX, C.c_uint64, C.POINTER(C.c_void_p)]),
    "sg_free": (C.c_int, [_CTX, C.c_void_p]),
    "sg_trim": (C.c_int, [_CTX]),
    "sg_mem_stats": (C.c_int, [_CTX, _U64P, _U64P, _U64P, _U64P]),
    "sg_memcpy_h2d": (C.c_int, [_CTX, C.c_void_p, C.c_void_p, C.c_uint64]),
    "sg_memcpy_d2h": (C.c_int, [_CTX, C.c_void_p, C.c_void_p, C.c_uint64]),
    "sg_memcpy_d2d": (C.c_int, [_CTX, C.c_void_p, C.c_void_p, C.c_uint64]),
    "sg_fill_u32": (C.c_int, [_CTX, C.c_void_p, C.c_uint32, C.c_uint64]),
    "sg_sync": (C.c_int, [_CTX]),
    "sg_stream": (C.c_void_p, [_CTX]),
    "sg_event_create": (C.c_int, [_CTX, C.POINTER(C.c_void_p)]),
    "sg_event_record": (C.c_int, [_CTX, C.c_void_p]),
    "sg_event_elapsed_ms": (C.c_int, [_CTX, C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]),
    "sg_event_destroy": (C.c_int, [_CTX, C.c_void_p]),
    "sg_last_error": (C.c_char_p, [_CTX]),
    "sg_last_oom": (C.c_int, [_CTX, _U64P, _U64P]),
    "sg_kernel_cache_size": (C.c_int, [_CTX]),
    "sg_map": (C.c_int, [_CTX, C.POINTER(sg_expr), C.c_int, _TP, C.c_int, _TP]),
    "sg_map_source": (C.c_int, [_CTX, C.POINTER(sg_expr), C.c_int, _TP, C.c_int, _TP, C.c_char_p, C.c_uint64, _I32P]),
    "sg_map_compile_only": (C.c_int, [C.c_char_p, C.c_char_p, C.c_uint64]),
    "sg_reduce": (C.c_int, [_CTX, C.c_int, _I32P, C.c_int, C.c_int, _TP, _TP]),
    "sg_reduce_arg": (C.c_int, [_CTX, C.c_int, C.c_int, _TP, _TP]),
    "sg_gather": (C.c_int, [_CTX, C.c_int, _TP, _TP, _TP]),
    "sg_scatter": (C.c_int, [_CTX, C.c_int, _TP, _TP, _TP]),
    "sg_unslice": (C.c_int, [_CTX, C.c_int, C.c_int64, _TP, _TP]),
    "sg_concat": (C.c_int, [_CTX, C.c_int, _TP, C.c_int, _TP]),
    "sg_gemm": (C.c_int, [_CTX, C.c_int, C.c_int, _TP, _TP, _TP, C.POINTER(sg_gemm_epilogue)]),
    "sg_gemm_noalloc": (C.c_int, [_CTX, C.c_int, C.c_int, _TP, _TP, _TP, C.POINTER(sg_gemm_epilogue)]),
    "sg_gemm_batched": (C.c_int, [_CTX, C.c_int, C.c_int, _TP, _TP, _TP, C.POINTER(sg_gemm_epilogue)]),
    "sg_matmul_strided": (C.c_int, [_CTX, _TP, _TP, _TP, C.POINTER(sg_gemm_epilogue)]),
    "sg_gemm_last_kernel_name": (C.c_int, [_CTX, C.c_char_p, C.c_uint64]),
    "sg_im2col": (C.c_int, [_CTX, _TP, _TP, _I32P, _I32P, _I32P, _I32P]),
    "sg_conv2d": (C.c_int, [_CTX, _TP, _TP, _TP, _I32P, _I32P, _I32P, C.POINTER(sg_gemm_epilogue)]),
    "sg_pool2d": (C.c_int, [_CTX, C.c_int, C.c_int, _TP, _TP, _I32P, _I32P, _I32P, _I32P]),
    "sg_col2im": (C.c_int, [_CTX, _TP, _TP, _I32P, _I32P, _I32P, _I32P]),
    "sg_softmax_lastaxis": (C.c_int, [_CTX, _TP, _TP, _TP]),
    "sg_softmax_cross_entropy": (C.c_int, [_CTX, _TP, _TP, _TP]),
    "sg_layer_norm_lastaxis": (C.c_int, [_CTX, _TP, _TP, _TP, C.c_float, _TP]),
    "sg_graph_begin": (C.c_int, [_CTX]),
    "sg_graph_end": (C.c_int, [_CTX, C.POINTER(C.c_void_p)]),
    "sg_graph_launch": (C.c_int, [_CTX, C.c_void_p]),
    "sg_graph_destroy": (C.c_int, [_CTX, C.c_void_p]),
    "sg_rand_uniform": (C.c_int, [_CTX, C.c_uint32, C.c_uint32, _TP]),
    "sg_rand_normal": (C.c_int, [_CTX, C.c_uint32, C.c_uint32, _TP]),
    "sg_adam_update": (C.c_int, [_CTX, C.c_int, _TP, _TP, _TP, _TP, _TP, C.POINTER(sg_adam_hyper)]),
    "sg_attention": (C.c_int, [_CTX, _TP, _TP, _TP, _TP, C.c_float, _TP]),
}

_lib = None


def lib():
    """The loaded library.  Raises if it has not been built (python -m sage_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m sage_amd.build` "
                "(hipcc --offload-arch=gfx950); there is no fallback path")
        l = C.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(l, name)  # AttributeError here = header and library disagree
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


class SageError(RuntimeError):
    def __init__(self, code, message, needed=None, total=None):
        super().__init__(f"[{['OK','OOM','DEVICE','SHAPE','DTYPE','ARG'][code]}] {message}")
        self.code = code
        self.needed = needed
        self.total = total


class ShapeError(SageError):
    pass


class DTypeError(SageError):
    pass


class OutOfMemory(SageError):
    pass


def check(ctx_handle, rc):
    if rc == OK:
        return
    msg = lib().sg_last_error(ctx_handle)
    msg = msg.decode() if msg else ""
    if rc == ERR_OOM:
        n, t = C.c_uint64(), C.c_uint64()
        lib().sg_last_oom(ctx_handle, C.byref(n), C.byref(t))
        raise OutOfMemory(rc, msg, n.value, t.value)
    cls = {ERR_SHAPE: ShapeError, ERR_DTYPE: DTypeError}.get(rc, SageError)
    raise cls(rc, msg)
