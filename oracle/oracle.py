"""CPU oracle: host tensors + the reference's operator compositions.  TEST INFRASTRUCTURE ONLY.

Nothing under sage_amd/ may import this module.  It drives oracle/libsage_oracle.so (the C
restatement of the reference's generated kernels) with numpy buffers and rebuilds, op for op, the
compositions the reference defines above its kernels:

  Shape algebra ......... shape.rs:45-54, 113-143, 183-279, 356-393
  Var layout methods .... ops/core.rs:200-523  (view/reshape organize first: core.rs:213-233, var.rs:506-512)
  map front-ends ........ ops/map.rs:412-456 (broadcast), 458-515 (dtype rules), 517-531 (scalar)
  reduce front-ends ..... ops/reduce.rs:50-140
  matmul ................ ops/gemm.rs:30-104
  conv / pools .......... ops/conv.rs:47-96, 143-165, 188-226
  nn .................... ops/nn.rs:33-100
  layers ................ layers.rs:208-247, 393-404, 423-463, 586-590
  BERT / ResNet ......... models/bert.rs, models/resnet.rs

Evaluation is eager and un-fused: every operator is one oracle "launch".  The reference fuses chains
of maps into one kernel (ops.rs:104-161); fusion changes only the launch count, never a value,
except that a fused comparison result stays a C `int` instead of being stored as `uint` first
(identical 0/1 values).  `fused_map` gives the fused form where a test or the CPU baseline wants
the reference's launch structure.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libsage_oracle.so")

MAX_RANK = 8
CHAR, SHORT, INT, LONG, UCHAR, USHORT, UINT, ULONG, FLOAT, HALF = range(10)
_NP = {FLOAT: np.float32, INT: np.int32, UINT: np.uint32}
_DT = {np.dtype(np.float32): FLOAT, np.dtype(np.int32): INT, np.dtype(np.uint32): UINT}

U = {n: i for i, n in enumerate(
    "copy abs neg recip log exp sqrt square erf sign ceil floor round sin sinh cos cosh tan tanh "
    "asin asinh acos acosh atan atanh not cast_int cast_float".split())}
B = {n: i for i, n in enumerate("add sub div mul mod pow min max and or eq ne gt ge lt le".split())}
K_INPUT, K_LITERAL, K_UNARY, K_BINARY, K_TERNARY = range(5)
R = {"sum": 0, "prod": 1, "max": 2, "min": 3}
INIT_REF_ZERO, INIT_IDENTITY = 0, 1


class CTensor(C.Structure):
    _fields_ = [("base", C.c_void_p), ("dtype", C.c_int32), ("rank", C.c_int32),
                ("extents", C.c_int64 * MAX_RANK), ("strides", C.c_int64 * MAX_RANK),
                ("offset", C.c_int64)]


class CExpr(C.Structure):
    _fields_ = [("kind", C.c_int32), ("op", C.c_int32), ("dtype", C.c_int32), ("bits", C.c_uint32)]


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
    return _lib


# ----------------------------------------------------------------------------- shape algebra
def default_strides(extents):
    size = 1
    for e in extents:
        size *= e
    out = []
    for e in extents:
        size //= e if e else 1
        out.append(size)
    return out


def union(s1, s2):
    """shape::union (shape.rs:356-393)."""
    s1, s2 = list(s1), list(s2)
    if s1 == s2:
        return s1
    longer, shorter = (s1, s2) if len(s1) > len(s2) else (s2, s1)
    u = longer[:len(longer) - len(shorter)] + shorter
    for i, (a, b) in enumerate(zip(u, longer)):
        if a != b:
            if a == 1:
                u[i] = b
            elif b != 1:
                raise ValueError("invalid broadcast")
    return u


class HT:
    """Host tensor: a flat 4-byte buffer plus (dtype, extents, strides, offset) — Tensor/TensorDesc."""

    def __init__(self, buf, dtype, extents, strides=None, offset=0):
        self.buf = buf  # 1-D numpy array, 4-byte elements
        self.dtype = dtype
        self.extents = [int(e) for e in extents]
        self.strides = [int(s) for s in (default_strides(self.extents) if strides is None else strides)]
        self.offset = int(offset)

    # -- construction / readback
    @staticmethod
    def from_numpy(a):
        a = np.ascontiguousarray(a)
        if a.dtype == np.float64:
            a = a.astype(np.float32)
        if a.dtype == np.int64:
            a = a.astype(np.int32)
        ext = list(a.shape) if a.ndim else [1]
        return HT(a.reshape(-1).copy(), _DT[a.dtype], ext)

    @staticmethod
    def empty(extents, dtype=FLOAT):
        n = int(np.prod(extents)) if len(extents) else 1
        return HT(np.zeros(n, dtype=_NP[dtype]), dtype, extents)

    def numpy(self):
        v = np.lib.stride_tricks.as_strided(self.buf[self.offset:], shape=self.extents,
                                            strides=[s * 4 for s in self.strides])
        return np.array(v)

    @property
    def rank(self):
        return len(self.extents)

    @property
    def size(self):
        n = 1
        for e in self.extents:
            n *= e
        return n

    def has_default_strides(self):  # shape.rs:134-143 (ignores offset)
        return self.strides == default_strides(self.extents)

    def ct(self):
        t = CTensor()
        t.base = self.buf.ctypes.data
        t.dtype = self.dtype
        t.rank = self.rank
        for i in range(self.rank):
            t.extents[i] = self.extents[i]
            t.strides[i] = self.strides[i]
        t.offset = self.offset
        return t

    def _like(self, extents, strides, offset):
        return HT(self.buf, self.dtype, extents, strides, offset)

    def _ax(self, a, bound=None):
        bound = self.rank if bound is None else bound
        return a + bound if a < 0 else a

    # -- zero-copy layout ops (core.rs:249-260, 315-317, 395-397, 434-436, 473-475, 520-522)
    def expand(self, extents):  # Shape::expand shape.rs:239-279
        extents = list(extents)
        ne, ns = list(self.extents), list(self.strides)
        for _ in range(len(extents) - len(ne)):
            ne.insert(0, 1)
            ns.insert(0, 0)
        for i, e in enumerate(extents):
            if ne[i] != e:
                if ne[i] == 1:
                    ne[i], ns[i] = e, 0
                else:
                    raise ValueError("invalid broadcast")
        return self._like(ne, ns, self.offset)

    def permute(self, axes):
        axes = [self._ax(a) for a in axes]
        return self._like([self.extents[a] for a in axes], [self.strides[a] for a in axes], self.offset)

    def transpose(self, a1, a2):
        a1, a2 = self._ax(a1), self._ax(a2)
        axes = list(range(self.rank))
        axes[a1], axes[a2] = a2, a1
        return self.permute(axes)

    def tr(self):
        return self.transpose(0, 1)

    def squeeze(self, axis):
        axis = self._ax(axis)
        e, s = list(self.extents), list(self.strides)
        del e[axis], s[axis]
        return self._like(e, s, self.offset)

    def unsqueeze(self, axis):  # Shape::insert: extent 1, stride 0 (shape.rs:190-195)
        axis = self._ax(axis, self.rank + 1)
        e, s = list(self.extents), list(self.strides)
        e.insert(axis, 1)
        s.insert(axis, 0)
        return self._like(e, s, self.offset)

    def slice(self, axis, start, end):  # select_range(start, end-1, axis) shape.rs:227-237
        axis = self._ax(axis)
        if end - 1 >= self.extents[axis]:
            raise IndexError("index out of bounds")
        e = list(self.extents)
        e[axis] = end - start
        return self._like(e, self.strides, self.offset + self.strides[axis] * start)

    def index(self, axis, i):  # var.rs:573-578
        return self.slice(axis, i, i + 1)

    # -- copies
    def organize(self):  # var.rs:506-512
        return self if self.has_default_strides() else unary("copy", self)

    def view(self, extents):  # core.rs:200-233 (+ -1 inference, shape.rs Extent::to_arr)
        extents = list(extents)
        if -1 in extents:
            known = 1
            for e in extents:
                if e != -1:
                    known *= e
            extents[extents.index(-1)] = self.size // known
        x = self.organize()
        n = 1
        for e in extents:
            n *= e
        if n != x.size:
            raise ValueError("incompatible size")
        return x._like(extents, default_strides(extents), x.offset)  # Reshape::compute adds offset


# ----------------------------------------------------------------------------- expression builder
class E:
    """Prefix expression tree -> sg_expr[] in the reference's order (ops.rs:116-130)."""

    def __init__(self, kind, op=0, args=(), dtype=0, bits=0):
        self.kind, self.op, self.args, self.dtype, self.bits = kind, op, args, dtype, bits

    @staticmethod
    def inp(i):
        return E(K_INPUT, i)

    @staticmethod
    def lit(value, dtype=FLOAT):
        bits = int(np.array(value, dtype=_NP[dtype]).view(np.uint32))
        return E(K_LITERAL, 0, (), dtype, bits)

    @staticmethod
    def un(name, a):
        return E(K_UNARY, U[name], (a,))

    @staticmethod
    def bin(name, a, b):
        return E(K_BINARY, B[name], (a, b))

    @staticmethod
    def cond(c, a, b):
        return E(K_TERNARY, 0, (c, a, b))

    def flat(self, out=None):
        out = [] if out is None else out
        out.append((self.kind, self.op, self.dtype, self.bits))
        for a in self.args:
            a.flat(out)
        return out

    def carray(self):
        f = self.flat()
        arr = (CExpr * len(f))()
        for i, (k, o, d, b) in enumerate(f):
            arr[i].kind, arr[i].op, arr[i].dtype, arr[i].bits = k, o, d, b
        return arr, len(f)


def unary_dtype(name, dt):  # map.rs:464-470
    if name in ("sign", "copy", "abs", "neg"):
        return dt
    if name == "not":
        return UINT
    if name == "cast_int":
        return INT
    return FLOAT


def binary_dtype(name, dt):  # map.rs:491-501
    return UINT if name in ("and", "or", "eq", "ne", "gt", "ge", "lt", "le") else dt


def fused_map(expr, inputs, out_dtype):
    """One `variadic` launch (map.rs:1141-1175)."""
    ext = inputs[0].extents if inputs else None
    for t in inputs:
        assert t.extents == ext
    y = HT.empty(ext, out_dtype)
    arr, n = expr.carray()
    ins = (CTensor * max(1, len(inputs)))(*[t.ct() for t in inputs])
    yt = y.ct()
    rc = lib().or_map(arr, n, ins, len(inputs), C.byref(yt))
    if rc:
        raise RuntimeError("or_map failed")
    return y


def scalar(value, extents, dtype=FLOAT):  # map.rs:517-531 nullary_map
    y = HT.empty(list(extents), dtype)
    arr, n = E.lit(value, dtype).carray()
    ins = (CTensor * 1)()
    yt = y.ct()
    assert lib().or_map(arr, n, ins, 0, C.byref(yt)) == 0
    return y


def _as_ht(v, like=None):
    if isinstance(v, HT):
        return v
    if isinstance(v, (int, np.integer)) and not isinstance(v, bool):
        return scalar(v, [1], INT)  # integer literals are Int (data.rs Scalar impls)
    return scalar(float(v), [1], FLOAT)


def broadcast(*xs):  # map.rs:412-456
    xs = [_as_ht(x) for x in xs]
    u = xs[0].extents
    for x in xs[1:]:
        u = union(u, x.extents)
    if len(xs) == 3:  # broadcast3 builds the union pairwise (map.rs:439-441)
        u = union(union(xs[0].extents, xs[1].extents), union(xs[1].extents, xs[2].extents))
    return [x if x.extents == list(u) else x.expand(u) for x in xs]


def unary(name, x):
    x = _as_ht(x)
    return fused_map(E.un(name, E.inp(0)), [x], unary_dtype(name, x.dtype))


def binary(name, a, b):
    a, b = broadcast(a, b)
    if a.dtype != b.dtype:
        raise TypeError("dtype mismatch")  # map.rs:489
    return fused_map(E.bin(name, E.inp(0), E.inp(1)), [a, b], binary_dtype(name, a.dtype))


def cond(c, a, b):  # map.rs:857-885
    c, a, b = broadcast(c, a, b)
    if a.dtype != b.dtype or c.dtype != UINT:
        raise TypeError("dtype mismatch")
    return fused_map(E.cond(E.inp(0), E.inp(1), E.inp(2)), [c, a, b], a.dtype)


# ----------------------------------------------------------------------------- reductions
def reduced_extents(extents, axes, preserve):  # reduce.rs:124-140
    out = []
    for i, e in enumerate(extents):
        if i not in axes:
            out.append(e)
        elif preserve:
            out.append(1)
    return out or [1]


def _axes(x, axes):
    if isinstance(axes, (int, np.integer)):
        axes = [axes]
    return [a + x.rank if a < 0 else a for a in axes]


def reduce(x, axes, preserve, op, init=INIT_REF_ZERO):
    axes = _axes(x, axes)
    y = HT.empty(reduced_extents(x.extents, axes, preserve), x.dtype)
    ax = (C.c_int32 * max(1, len(axes)))(*axes)
    xt, yt = x.ct(), y.ct()
    if lib().or_reduce(R[op], ax, len(axes), init, C.byref(xt), C.byref(yt)):
        raise RuntimeError("or_reduce failed")
    return y


def rsum(x, axes, preserve=False):
    return reduce(x, axes, preserve, "sum")


def rmax(x, axes, preserve=False, init=INIT_REF_ZERO):
    return reduce(x, axes, preserve, "max", init)


def rmin(x, axes, preserve=False, init=INIT_REF_ZERO):
    return reduce(x, axes, preserve, "min", init)


def rprod(x, axes, preserve=False, init=INIT_REF_ZERO):
    return reduce(x, axes, preserve, "prod", init)


def mean(x, axes, preserve=False):  # reduce.rs:59-71
    axes = _axes(x, axes)
    size = 1
    for a in axes:
        size *= x.extents[a]
    r = rsum(x, axes, preserve)
    return binary("div", r, scalar(float(size), r.extents))


def var(x, axes, preserve=False):  # reduce.rs:73-82
    axes = _axes(x, axes)
    return binary("sub", mean(unary("square", x), axes, preserve), unary("square", mean(x, axes, preserve)))


def reduce_arg(x, axis, preserve, op):
    axis = _axes(x, axis)[0]
    y = HT.empty(reduced_extents(x.extents, [axis], preserve), UINT)
    xt, yt = x.ct(), y.ct()
    if lib().or_reduce_arg(0 if op == "max" else 1, axis, C.byref(xt), C.byref(yt)):
        raise RuntimeError("or_reduce_arg failed")
    return y


def argmax(x, axis, preserve=False):
    return reduce_arg(x, axis, preserve, "max")


def argmin(x, axis, preserve=False):
    return reduce_arg(x, axis, preserve, "min")


# ----------------------------------------------------------------------------- indexing
def gather(x, ind, axis):  # core.rs:620-653
    axis = _axes(x, axis)[0]
    assert x.rank == ind.rank
    y = HT.empty(ind.extents, x.dtype)
    xt, it, yt = x.ct(), ind.ct(), y.ct()
    if lib().or_gather(axis, C.byref(xt), C.byref(it), C.byref(yt)):
        raise RuntimeError("or_gather failed")
    return y


def scatter(x, ind, axis, extents):  # core.rs:721-762
    axis = _axes(x, axis)[0]
    y = HT.empty(list(extents), x.dtype)
    xt, it, yt = x.ct(), ind.ct(), y.ct()
    if lib().or_scatter(axis, C.byref(xt), C.byref(it), C.byref(yt)):
        raise RuntimeError("or_scatter failed")
    return y


def unslice(x, axis, start, end):  # core.rs:525-551
    axis = _axes(x, axis)[0]
    assert end >= start + x.extents[axis]
    ext = list(x.extents)
    ext[axis] = end
    y = HT.empty(ext, x.dtype)
    xt, yt = x.ct(), y.ct()
    assert lib().or_unslice(axis, C.c_int64(start), C.byref(xt), C.byref(yt)) == 0
    return y


def concat(xs, axis):  # core.rs:836-871
    axis = _axes(xs[0], axis)[0]
    ext = list(xs[0].extents)
    ext[axis] = sum(x.extents[axis] for x in xs)
    y = HT.empty(ext, xs[0].dtype)
    ins = (CTensor * len(xs))(*[x.ct() for x in xs])
    yt = y.ct()
    assert lib().or_concat(axis, ins, len(xs), C.byref(yt)) == 0
    return y


# ----------------------------------------------------------------------------- GEMM
def gemm(a, b, ta=False, tb=False):  # gemm.rs:106-140
    a, b = a.organize(), b.organize()
    m = a.extents[1 if ta else 0]
    n = b.extents[0 if tb else 1]
    y = HT.empty([m, n], FLOAT)
    at, bt, yt = a.ct(), b.ct(), y.ct()
    if lib().or_gemm(int(ta), int(tb), C.byref(at), C.byref(bt), C.byref(yt)):
        raise RuntimeError("or_gemm failed")
    return y


def gemm_batched(a, b, ta=False, tb=False):  # gemm.rs:253-290
    a, b = a.organize(), b.organize()
    m = a.extents[2 if ta else 1]
    n = b.extents[1 if tb else 2]
    y = HT.empty([a.extents[0], m, n], FLOAT)
    at, bt, yt = a.ct(), b.ct(), y.ct()
    if lib().or_gemm_batched(int(ta), int(tb), C.byref(at), C.byref(bt), C.byref(yt)):
        raise RuntimeError("or_gemm_batched failed")
    return y


def matmul(x1, x2):  # gemm.rs:30-51
    ext = x1.extents[:-1] + x2.extents[1:]
    a = x1.view([x1.size // x1.extents[-1], x1.extents[-1]])
    b = x2.view([x2.extents[0], x2.size // x2.extents[0]])
    return gemm(a, b).view(ext)


def matmul_batched(x1, x2):  # gemm.rs:53-104
    batch = []
    for i in range(min(x1.rank - 2, x2.rank - 2)):
        if x1.extents[i] == x2.extents[i]:
            batch.append(x1.extents[i])
        else:
            break
    bl = len(batch)
    if bl == 0:
        raise ValueError("batch dim incorrect!")
    bs = int(np.prod(batch))
    ext = batch + x1.extents[bl:x1.rank - 1] + x2.extents[bl + 1:]
    a = x1.view([bs, x1.size // (x1.extents[-1] * bs), x1.extents[-1]])
    b = x2.view([bs, x2.extents[bl], x2.size // (x2.extents[bl] * bs)])
    return gemm_batched(a, b).view(ext)


# ----------------------------------------------------------------------------- conv / pools
def _pair(v):
    return [v, v] if isinstance(v, (int, np.integer)) else list(v)


def conv_size(size, ker, stride, pad, dil):  # conv.rs:47-59
    return [(size[i] + 2 * pad[i] - dil[i] * (ker[i] - 1) - 1) // stride[i] + 1 for i in range(2)]


def im2col(x, ker, stride, pad, dil):  # conv.rs:188-226 ; pairs are [w, h]
    ker, stride, pad, dil = _pair(ker), _pair(stride), _pair(pad), _pair(dil)
    x = x.organize()
    n, h, w, c = x.extents
    col = conv_size([w, h], ker, stride, pad, dil)
    y = HT.empty([n, col[1], col[0], ker[1], ker[0], c], x.dtype)
    arr = lambda v: (C.c_int32 * 2)(*v)
    xt, yt = x.ct(), y.ct()
    if lib().or_im2col(C.byref(xt), C.byref(yt), arr(ker), arr(stride), arr(pad), arr(dil)):
        raise RuntimeError("or_im2col failed")
    return y


def col2im(x, img_size, ker, stride, pad, dil):  # conv.rs:229-264 ; img_size and pairs are [w, h]
    ker, stride, pad, dil = _pair(ker), _pair(stride), _pair(pad), _pair(dil)
    x = x.organize()
    n, c = x.extents[0], x.extents[5]
    y = HT.empty([n, img_size[1], img_size[0], c], x.dtype)
    arr = lambda v: (C.c_int32 * 2)(*v)
    xt, yt = x.ct(), y.ct()
    if lib().or_col2im(C.byref(xt), C.byref(yt), arr(ker), arr(stride), arr(pad), arr(dil)):
        raise RuntimeError("or_col2im failed")
    return y


def conv_2d(x, filt, stride, pad, dil):  # conv.rs:61-96
    kh, kw, cin, cout = filt.extents
    col = im2col(x, [kw, kh], stride, pad, dil)
    n, ch, cw = col.extents[:3]
    col = col.view([n * ch * cw, kh * kw * cin])
    f = filt.view([kh * kw * cin, cout])
    return matmul(col, f).view([n, ch, cw, cout])


def conv_transpose_2d(x, filt, stride, pad, dil):  # conv.rs:98-140 (output size: conv.rs:33-45)
    n, h, w, cin = x.extents
    kh, kw, cout = filt.extents[0], filt.extents[1], filt.extents[2]
    f = filt.permute([2, 0, 1, 3]).organize().view([cin, kh * kw * cout])
    col = matmul(x.view([n * h * w, cin]), f).view([n, h, w, kh, kw, cout])
    ker, stride, pad, dil = [kw, kh], _pair(stride), _pair(pad), _pair(dil)
    out = [(s - 1) * st - 2 * p + d * (k - 1) for s, k, st, p, d in zip([w, h], ker, stride, pad, dil)]
    return col2im(col, out, ker, stride, pad, dil)


def max_pool_2d(x, ker, stride, pad, dil):  # conv.rs:155-165
    return rmax(im2col(x, ker, stride, pad, dil), [3, 4], False)


def avg_pool_2d(x, ker, stride, pad, dil):  # conv.rs:143-153
    return mean(im2col(x, ker, stride, pad, dil), [3, 4], False)


# ----------------------------------------------------------------------------- nn (nn.rs:33-100)
def relu(x):
    return binary("mul", unary("cast_float", binary("gt", x, 0.0)), x)


def softmax(x, axes):
    axes = _axes(x, axes)
    xm = rmax(x, axes, True)
    y = unary("exp", binary("sub", x, xm))
    s = rsum(y, axes, True)
    return binary("div", y, s)


def log_sum_exp(x, axes):
    axes = _axes(x, axes)
    c = rmax(x, axes, True)
    return binary("add", unary("log", rsum(unary("exp", binary("sub", x, c)), axes, True)), c)


def softmax_cross_entropy(x, labels):
    log_z = binary("sub", x, log_sum_exp(x, 1))
    log_p = gather(log_z, labels, 1)
    return unary("neg", rsum(log_p, 1, False))


def layer_norm(x, axes, gamma, beta, eps):
    axes = _axes(x, axes)
    m = mean(x, axes, True)
    v = var(x, axes, True)
    xc = binary("div", binary("sub", x, m), unary("sqrt", binary("add", v, float(eps))))
    return binary("add", binary("mul", xc, gamma), beta)


def accuracy(logits, labels):  # metric.rs:4-16
    am = argmax(logits, 1, True)
    hit = binary("eq", am, labels)
    return unary("cast_float", rsum(hit, 0, False)).numpy() / logits.extents[0]


# ----------------------------------------------------------------------------- layers
def dense(x, w, b):  # layers.rs:243-247
    return binary("add", matmul(x, w), b)


def conv2d_layer(x, w, b, stride, pad, dil=1):  # layers.rs:393-404
    return binary("add", conv_2d(x, w, _pair(stride), _pair(pad), _pair(dil)), b)


def embedding(weight, idx):  # layers.rs:423-463
    dim = weight.extents[1]
    if idx.rank > 1:
        b, l = idx.extents[0], idx.extents[1]
        i = idx.view([b * l, 1]).expand([b * l, dim])
        return gather(weight, i, 0).view([b, l, dim])
    l = idx.extents[0]
    i = idx.view([l, 1]).expand([l, dim])
    return gather(weight, i, 0).view([l, dim])


def adaptive_avg_pool_2d(x, out):  # layers.rs:141-153
    iw, ih = x.extents[2], x.extents[1]
    ow, oh = out
    stride = [iw // ow, ih // oh]
    ker = [iw - (ow - 1) * stride[0], ih - (oh - 1) * stride[1]]
    return avg_pool_2d(x, ker, stride, [0, 0], [1, 1])


# ----------------------------------------------------------------------------- BERT (models/bert.rs)
def bert_attention(x, mask, p, heads, act_eps=1e-5):
    """MultiHeadAttention::pass (bert.rs:250-280).  p: dict of HT weights."""
    n, l, e = x.extents
    d = e // heads
    q = dense(x, p["wq"], p["bq"])
    k = dense(x, p["wk"], p["bk"])
    v = dense(x, p["wv"], p["bv"])
    sep = lambda t: t.view([n, l, heads, d]).transpose(2, 1)  # bert.rs:282-291
    q, k, v = sep(q), sep(k), sep(v)
    att = binary("div", matmul_batched(q, k.transpose(-1, -2)), float(np.sqrt(np.float32(d))))
    ext_mask = binary("mul", binary("add", unary("neg", mask.view([n, 1, 1, l])), 1.0), -1e5)  # bert.rs:304-314
    att = softmax(binary("add", att, ext_mask), [3])
    av = matmul_batched(att, v)
    av = av.transpose(2, 1).view([n, l, heads * d])  # merge_heads bert.rs:293-302
    y = dense(av, p["wo"], p["bo"])
    return layer_norm(binary("add", y, x), [2], p["ln1_g"], p["ln1_b"], act_eps)


def bert_layer(x, mask, p, heads, act="relu", eps=1e-5):
    """BertLayer::pass (bert.rs:199-203).  act='relu' and eps=1e-5 are what the reference runs
    (bert.rs:192, layers.rs:588); act='gelu' gives the erf-GELU variant from the same ops."""
    h1 = bert_attention(x, mask, p, heads, eps)
    u = dense(h1, p["w1"], p["b1"])
    if act == "relu":
        u = relu(u)
    else:  # 0.5*x*(1+erf(x/sqrt(2)))
        u = binary("mul", binary("mul", u, 0.5),
                   binary("add", unary("erf", binary("div", u, float(np.sqrt(np.float32(2.0))))), 1.0))
    f = dense(u, p["w2"], p["b2"])
    return layer_norm(binary("add", f, h1), [2], p["ln2_g"], p["ln2_b"], eps)


def bert_embedding(ids, p, eps=1e-5, segment_ids=None):  # BertEmbedding::pass bert.rs:128-139
    """word + position embeddings -> LayerNorm.  The reference has no segment table (bert.rs:97-102);
    when p holds "seg_emb" and segment_ids is given, its rows are added the same way before the
    LayerNorm (the benchmark's configuration variant)."""
    l = ids.extents[1]
    pos = HT.from_numpy(np.arange(l, dtype=np.uint32))
    we = embedding(p["word_emb"], ids)
    pe = embedding(p["pos_emb"], pos)
    e = binary("add", we, pe)
    if segment_ids is not None and "seg_emb" in p:
        e = binary("add", e, embedding(p["seg_emb"], segment_ids))
    return layer_norm(e, [2], p["emb_g"], p["emb_b"], eps)


def bert_forward(ids, mask, p, heads, act="relu", eps=1e-5, cls_index=1, segment_ids=None, return_hidden=False):
    """Bert::pass (bert.rs:72-81): classifier on token index 1 (cls_index=0, act='gelu', eps=1e-12 and a
    segment table give the benchmark's configuration variant from the same operators)."""
    x = bert_embedding(ids, p, eps, segment_ids)
    for lp in p["layers"]:
        x = bert_layer(x, mask, lp, heads, act, eps)
    cls = x.index(1, cls_index).squeeze(1)
    y = dense(cls, p["wc"], p["bc"])
    return (y, x) if return_hidden else y


# ----------------------------------------------------------------------------- ResNet (models/resnet.rs)
def resnet_basic(x, p, stride):  # BasicLayer::pass resnet.rs:270-279
    y = conv2d_layer(x, p["w1"], p["b1"], stride, 1)
    y = relu(y)
    y = conv2d_layer(y, p["w2"], p["b2"], 1, 1)
    sc = conv2d_layer(x, p["wd"], p["bd"], stride, 0) if "wd" in p else x
    return relu(binary("add", y, sc))


def resnet18_forward(x, p):  # ResNet::new resnet.rs:75-104 with d18
    y = conv2d_layer(x, p["w0"], p["b0"], 2, 3)
    y = relu(y)
    y = max_pool_2d(y, [3, 3], [2, 2], [1, 1], [1, 1])
    for blk in p["blocks"]:
        y = resnet_basic(y, blk, blk["stride"])
    y = adaptive_avg_pool_2d(y, [1, 1])
    y = y.view([y.extents[0], -1])
    return dense(y, p["wfc"], p["bfc"])


def rand_uniform(extents, seed_x, seed_y):  # rand.rs:62-97
    y = HT.empty(list(extents), FLOAT)
    yt = y.ct()
    lib().or_rand_uniform(C.c_uint32(seed_x), C.c_uint32(seed_y), C.byref(yt))
    return y


def rand_normal(extents, seed_x, seed_y):  # rand.rs:105-146
    y = HT.empty(list(extents), FLOAT)
    yt = y.ct()
    lib().or_rand_normal(C.c_uint32(seed_x), C.c_uint32(seed_y), C.byref(yt))
    return y


def num_threads():
    return lib().or_num_threads()
