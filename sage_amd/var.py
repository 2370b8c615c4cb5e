"""Lazy variables and the operator front-end: host-side mirror of var.rs, ops/*.rs and the parts of
session.rs that decide what one kernel launch covers.

`Var` is a node of a lazily built graph (var.rs:33-42); nothing touches the device until
`Var.eval(ctx)` (var.rs:338-352).  The front-end functions keep the reference's names, argument
meaning, dtype rules and assert sites (raising instead of panicking).  Evaluation differs from the
reference's `Program::compile`/`Routine::exec` (session.rs:62-206, 514-673) in how much one launch
covers, never in values:

  * chains of maps become ONE run-time-built kernel, as in Operator::fuse (ops.rs:104-161), and
    Expand(literal) folds into the literal (ops.rs:145-155);
  * bias / scale / activation / residual maps that directly consume a GEMM are folded into the
    GEMM's epilogue instead of being separate full-size passes (layers.rs:243-247, nn.rs:33-40);
  * matmul_batched consumes permuted (strided) operands in place and can write a permuted result
    in place, instead of organize() copies around the kernel (gemm.rs:258-259, bert.rs:282-302);
  * softmax / layer_norm / softmax_cross_entropy over the last axis run as one fused row kernel
    instead of the 4-10 launches of their compositions (nn.rs:42-100).
`set_fusion(False)` turns all of that off: every operator is then launched on its own, which is what
the parity tests compare the fused results against.
"""
import ctypes as C
import os
import time

import numpy as np

from . import abi
from .shape import Shape, default_strides, infer_extents, norm_axes, norm_axis, union
from .tensor import FLOAT, INT, UINT, Context, Tensor

_FUSION = {"on": True}
THRES = 5  # session.rs:75


# Parameters may be rewritten in place (optimizers do); derived data that the evaluator caches, the
# concatenated weights of sibling Dense layers, is rebuilt when this counter has moved since it was made.
from .tensor import _PARAM_EPOCH  # noqa: E402  (shared counter, also bumped by Tensor.copy_from_numpy)


def params_changed():
    """Tell cached derived data that parameter values may have changed."""
    _PARAM_EPOCH[0] += 1


def set_fusion(on):
    _FUSION["on"] = bool(on)


def fusion_enabled():
    return _FUSION["on"]


MAP_OPS = ("literal", "unary", "binary", "cond")
GEMM_OPS = ("gemm", "gemm_batched", "matmul_nd")


class Var:
    """var.rs:33-42.  op == "data" holds a Tensor (Origin::Data); anything else is an Operation."""

    __slots__ = ("shape", "dtype", "op", "inputs", "attrs", "value", "label", "__weakref__")

    def __init__(self, shape, dtype, op, inputs=(), attrs=None, value=None):
        self.shape = shape
        self.dtype = dtype
        self.op = op
        self.inputs = tuple(inputs)
        self.attrs = attrs or {}
        self.value = value  # Tensor once evaluated (ctx.data in the reference, context.rs:27)
        self.label = None

    # ---- constructors
    @staticmethod
    def new(tensor):
        return Var(tensor.shape.copy(), tensor.dtype, "data", value=tensor)

    @staticmethod
    def empty(extents, dtype=FLOAT):
        return Var(Shape(extents), dtype, "data")

    def set(self, tensor):
        """Var::set (var.rs:371-378)."""
        if self.op != "data":
            raise TypeError("can only assign tensor to the data variable")
        self.value = tensor
        self.shape = tensor.shape.copy()
        self.dtype = tensor.dtype
        params_changed()

    def name(self, label):
        self.label = label
        return self

    # ---- properties
    @property
    def extents(self):
        return self.shape.extents

    @property
    def rank(self):
        return self.shape.rank

    def size(self):
        return self.shape.size()

    def extent(self, axis):
        return self.shape.extents[norm_axis(axis, self.rank)]

    def is_data(self):
        return self.op == "data"

    def eval(self, ctx):
        """Var::eval (var.rs:338-352)."""
        if self.op == "data":
            if self.value is None:
                raise RuntimeError("cannot evaluate empty var")
            return self.value
        return evaluate(ctx, [self])[0]

    def grad(self, y):
        """Var::grad (var.rs:326-334): the gradient of `y` with respect to this variable."""
        from .grad import grad
        return grad(into_var(y), [self])[0]

    # ---- fluent API (var.rs:382-700)
    def copy(self): return unary_map(self, "copy")
    def abs(self): return unary_map(self, "abs")
    def recip(self): return unary_map(self, "recip")
    def log(self): return unary_map(self, "log")
    def exp(self): return unary_map(self, "exp")
    def sqrt(self): return unary_map(self, "sqrt")
    def square(self): return unary_map(self, "square")
    def erf(self): return unary_map(self, "erf")
    def sign(self): return unary_map(self, "sign")
    def ceil(self): return unary_map(self, "ceil")
    def floor(self): return unary_map(self, "floor")
    def round(self): return unary_map(self, "round")
    def sin(self): return unary_map(self, "sin")
    def sinh(self): return unary_map(self, "sinh")
    def cos(self): return unary_map(self, "cos")
    def cosh(self): return unary_map(self, "cosh")
    def tan(self): return unary_map(self, "tan")
    def tanh(self): return unary_map(self, "tanh")
    def asin(self): return unary_map(self, "asin")
    def asinh(self): return unary_map(self, "asinh")
    def acos(self): return unary_map(self, "acos")
    def acosh(self): return unary_map(self, "acosh")
    def atan(self): return unary_map(self, "atan")
    def atanh(self): return unary_map(self, "atanh")
    def int(self): return unary_map(self, "cast_int")
    def float(self): return unary_map(self, "cast_float")
    def pow(self, x): return binary_map(self, x, "pow")
    def minimum(self, x): return binary_map(self, x, "min")
    def maximum(self, x): return binary_map(self, x, "max")
    def modular(self, x): return binary_map(self, x, "mod")

    def organize(self):
        """var.rs:506-512."""
        return self if self.shape.has_default_strides() else self.copy()

    def reshape(self, shape): return reshape(self, shape)
    def view(self, extents): return view(self, extents)
    def expand(self, extents): return expand(self, extents)
    def tr(self): return transpose(self, 0, 1)
    def transpose(self, a1, a2): return transpose(self, a1, a2)
    def permute(self, axes): return permute(self, axes)
    def squeeze(self, axis): return squeeze(self, axis)
    def unsqueeze(self, axis): return unsqueeze(self, axis)
    def index(self, axis, i): return slice_(self, axis, i, i + 1)
    def slice(self, axis, start, end): return slice_(self, axis, start, end)
    def unslice(self, axis, start, end): return unslice(self, axis, start, end)
    def gather(self, idx, axis): return gather(self, idx, axis)
    def scatter(self, idx, axis, extents): return scatter(self, idx, axis, extents)
    def matmul(self, x): return matmul(self, x)
    def matmul_batched(self, x): return matmul_batched(self, x)
    def sum(self, axes, preserve_axes=False): return reduce(self, axes, preserve_axes, "sum")
    def prod(self, axes, preserve_axes=False): return reduce(self, axes, preserve_axes, "prod")
    def max(self, axes, preserve_axes=False): return reduce(self, axes, preserve_axes, "max")
    def min(self, axes, preserve_axes=False): return reduce(self, axes, preserve_axes, "min")
    def mean(self, axes, preserve_axes=False): return mean(self, axes, preserve_axes)
    def var(self, axes, preserve_axes=False): return var(self, axes, preserve_axes)
    def argmax(self, axis, preserve_axes=False): return reduce_arg(self, axis, preserve_axes, "max")
    def argmin(self, axis, preserve_axes=False): return reduce_arg(self, axis, preserve_axes, "min")

    def __add__(self, o): return binary_map(self, o, "add")
    def __radd__(self, o): return binary_map(o, self, "add")
    def __sub__(self, o): return binary_map(self, o, "sub")
    def __rsub__(self, o): return binary_map(o, self, "sub")
    def __mul__(self, o): return binary_map(self, o, "mul")
    def __rmul__(self, o): return binary_map(o, self, "mul")
    def __truediv__(self, o): return binary_map(self, o, "div")
    def __rtruediv__(self, o): return binary_map(o, self, "div")
    def __neg__(self): return unary_map(self, "neg")

    def __repr__(self):
        return f"{self.label or 'unnamed'}({self.op}) -> {self.shape!r} dtype={self.dtype}"


def into_var(v):
    """Variable::into_var (var.rs:795-861): tensors wrap, scalars become scalar(v, [1])."""
    if isinstance(v, Var):
        return v
    if isinstance(v, Tensor):
        return Var.new(v)
    if isinstance(v, (bool, np.bool_)):
        raise TypeError("bool is not a Scalar")
    if isinstance(v, (int, np.integer)):
        return scalar(int(v), [1], INT)
    if isinstance(v, (float, np.floating)):
        return scalar(float(v), [1], FLOAT)
    raise TypeError(f"cannot make a Var from {type(v).__name__}")


# ----------------------------------------------------------------------------- maps (ops/map.rs)
def scalar(val, extents, dtype=None):
    """map.rs:517-531.  A Python float is a Float literal, a Python int an Int literal."""
    if dtype is None:
        dtype = INT if isinstance(val, (int, np.integer)) else FLOAT
    if isinstance(extents, int):
        extents = [extents]
    return Var(Shape(extents), dtype, "literal", attrs={"value": val})


def broadcast(*xs):
    """map.rs:412-456."""
    xs = [into_var(x) for x in xs]
    if len(xs) == 2:
        u = union(xs[0].extents, xs[1].extents)
    else:
        u = union(union(xs[0].extents, xs[1].extents), union(xs[1].extents, xs[2].extents))
    return [x if x.extents == list(u) else expand(x, u) for x in xs]


def unary_dtype(name, dt):
    """map.rs:464-470."""
    if name in ("sign", "copy", "abs", "neg"):
        return dt
    if name == "not":
        return UINT
    if name == "cast_int":
        return INT
    return FLOAT


def unary_map(x, name):
    x = into_var(x)
    if name not in abi.U:
        raise ValueError(f"unknown unary map {name}")
    return Var(Shape(x.extents), unary_dtype(name, x.dtype), "unary", [x], {"name": name})


def binary_map(x1, x2, name):
    """map.rs:472-515."""
    x1, x2 = broadcast(x1, x2)
    if x1.dtype != x2.dtype:
        raise abi.DTypeError(abi.ERR_DTYPE, "binary map operands differ in dtype (map.rs:489)")
    dt = UINT if name in ("and", "or", "eq", "ne", "gt", "ge", "lt", "le") else x1.dtype
    return Var(Shape(x1.extents), dt, "binary", [x1, x2], {"name": name})


def cond(c, x1, x2):
    """map.rs:857-885."""
    c, x1, x2 = broadcast(c, x1, x2)
    if x1.dtype != x2.dtype:
        raise abi.DTypeError(abi.ERR_DTYPE, "cond branches differ in dtype (map.rs:869)")
    if c.dtype != UINT:
        raise abi.DTypeError(abi.ERR_DTYPE, "cond condition must be uint (map.rs:870)")
    return Var(Shape(x1.extents), x1.dtype, "cond", [c, x1, x2])


def _mk_unary(name):
    return lambda x: unary_map(x, name)


def _mk_binary(name):
    return lambda a, b: binary_map(a, b, name)


copy, abs_, neg, recip, log, exp, sqrt, square, erf, sign = (_mk_unary(n) for n in
    ("copy", "abs", "neg", "recip", "log", "exp", "sqrt", "square", "erf", "sign"))
ceil, floor, round_, sin, sinh, cos, cosh, tan, tanh = (_mk_unary(n) for n in
    ("ceil", "floor", "round", "sin", "sinh", "cos", "cosh", "tan", "tanh"))
asin, asinh, acos, acosh, atan, atanh, logical_not = (_mk_unary(n) for n in
    ("asin", "asinh", "acos", "acosh", "atan", "atanh", "not"))
add, sub, div, mul, modular, pow_, minimum, maximum = (_mk_binary(n) for n in
    ("add", "sub", "div", "mul", "mod", "pow", "min", "max"))
logical_and, logical_or, eq, ne, gt, ge, lt, le = (_mk_binary(n) for n in
    ("and", "or", "eq", "ne", "gt", "ge", "lt", "le"))


# ----------------------------------------------------------------------------- layout (ops/core.rs)
def reshape(x, shape):
    """core.rs:213-233: organize first, then a pure descriptor change."""
    x = into_var(x).organize()
    if x.size() != shape.size():
        raise abi.ShapeError(abi.ERR_SHAPE, "incompatible size")
    return Var(shape.copy(), x.dtype, "reshape", [x])


def view(x, extents):
    """core.rs:200-211."""
    x = into_var(x)
    if isinstance(extents, int):
        extents = [extents]
    return reshape(x, Shape(infer_extents(extents, x.size())))


def expand(x, extents):
    """core.rs:263-322; Expand(literal) is folded as ops.rs:145-155 does."""
    x = into_var(x)
    sh = x.shape.expand(list(extents))
    if x.op == "literal" and _FUSION["on"]:
        return Var(Shape(sh.extents), x.dtype, "literal", attrs=dict(x.attrs))
    return Var(sh, x.dtype, "expand", [x])


def permute(x, axes):
    """core.rs:358-398."""
    x = into_var(x)
    axes = norm_axes(list(axes), x.rank)
    if sorted(axes) != list(range(x.rank)):
        raise abi.ShapeError(abi.ERR_SHAPE, "permute needs every axis exactly once")
    return Var(x.shape.permute(axes), x.dtype, "permute", [x], {"axes": axes})


def transpose(x, a1, a2):
    """core.rs:330-356."""
    x = into_var(x)
    a1, a2 = norm_axis(a1, x.rank), norm_axis(a2, x.rank)
    axes = list(range(x.rank))
    axes[a1], axes[a2] = a2, a1
    return permute(x, axes)


def tr(x):
    return transpose(x, 0, 1)


def squeeze(x, axis):
    """core.rs:400-437."""
    x = into_var(x)
    axis = norm_axis(axis, x.rank)
    return Var(x.shape.remove(axis), x.dtype, "squeeze", [x], {"axis": axis})


def unsqueeze(x, axis):
    """core.rs:439-476."""
    x = into_var(x)
    axis = norm_axis(axis, x.rank + 1)
    return Var(x.shape.insert(axis), x.dtype, "unsqueeze", [x], {"axis": axis})


def slice_(x, axis, start, end):
    """core.rs:478-523."""
    x = into_var(x)
    axis = norm_axis(axis, x.rank)
    if end <= start or end > x.extents[axis]:
        raise abi.ShapeError(abi.ERR_SHAPE, "index out of bounds")
    return Var(x.shape.select_range(start, end - 1, axis), x.dtype, "slice", [x], {"axis": axis, "start": start, "end": end})


def unslice(x, axis, start, end):
    """core.rs:525-551."""
    x = into_var(x)
    axis = norm_axis(axis, x.rank)
    if end < start + x.extents[axis]:
        raise abi.ShapeError(abi.ERR_SHAPE, "unslice window does not fit (core.rs:534)")
    ext = list(x.extents)
    ext[axis] = end
    return Var(Shape(ext), x.dtype, "unslice", [x], {"axis": axis, "start": start})


def gather(x, ind, axis):
    """core.rs:620-653."""
    x, ind = into_var(x), into_var(ind)
    axis = norm_axis(axis, x.rank)
    if x.rank != ind.rank:
        raise abi.ShapeError(abi.ERR_SHAPE, "gather: ranks differ (core.rs:631)")
    return Var(Shape(ind.extents), x.dtype, "gather", [x, ind], {"axis": axis})


def scatter(x, ind, axis, extents):
    """core.rs:721-762."""
    x, ind = into_var(x), into_var(ind)
    axis = norm_axis(axis, x.rank)
    extents = list(extents)
    if len(extents) != x.rank or x.rank != ind.rank:
        raise abi.ShapeError(abi.ERR_SHAPE, "scatter: ranks differ (core.rs:736-737)")
    return Var(Shape(extents), x.dtype, "scatter", [x, ind], {"axis": axis})


def concat(xs, axis):
    """core.rs:836-871."""
    xs = [into_var(x) for x in xs]
    axis = norm_axis(axis, xs[0].rank)
    ext = list(xs[0].extents)
    total = 0
    for v in xs:
        if v.rank != xs[0].rank or v.extents[:axis] != ext[:axis] or v.extents[axis + 1:] != ext[axis + 1:]:
            raise abi.ShapeError(abi.ERR_SHAPE, "not in the same shape")
        total += v.extents[axis]
    ext[axis] = total
    return Var(Shape(ext), xs[0].dtype, "concat", xs, {"axis": axis})


# ----------------------------------------------------------------------------- reductions (ops/reduce.rs)
def reduced_extents(extents, axes, preserve):
    """reduce.rs:124-140."""
    out = []
    for i, e in enumerate(extents):
        if i not in axes:
            out.append(e)
        elif preserve:
            out.append(1)
    return out or [1]


def reduce(x, axes, preserve_axes, op, init="ref_zero"):
    """reduce.rs:224-256.  init="ref_zero" is the reference's accumulator (literal 0 for every op,
    reduce.rs:282); init="identity" uses the mathematical identity instead."""
    x = into_var(x)
    axes = norm_axes(axes, x.rank)
    return Var(Shape(reduced_extents(x.extents, axes, preserve_axes)), x.dtype, "reduce", [x],
               {"op": op, "axes": axes, "init": init})


def sum_(x, axes, preserve_axes=False): return reduce(x, axes, preserve_axes, "sum")
def prod(x, axes, preserve_axes=False): return reduce(x, axes, preserve_axes, "prod")
def max_(x, axes, preserve_axes=False): return reduce(x, axes, preserve_axes, "max")
def min_(x, axes, preserve_axes=False): return reduce(x, axes, preserve_axes, "min")


def mean(x, axes, preserve_axes=False):
    """reduce.rs:59-71."""
    x = into_var(x)
    axes = norm_axes(axes, x.rank)
    size = 1
    for a in axes:
        size *= x.extents[a]
    r = reduce(x, axes, preserve_axes, "sum")
    return r / scalar(float(size), r.extents)


def var(x, axes, preserve_axes=False):
    """reduce.rs:73-82."""
    x = into_var(x)
    axes = norm_axes(axes, x.rank)
    return x.square().mean(axes, preserve_axes) - x.mean(axes, preserve_axes).square()


def reduce_arg(x, axis, preserve_axes, op):
    """reduce.rs:327-350."""
    x = into_var(x)
    axis = norm_axis(axis, x.rank)
    return Var(Shape(reduced_extents(x.extents, [axis], preserve_axes)), UINT, "reduce_arg", [x], {"op": op, "axis": axis})


def argmax(x, axis, preserve_axes=False): return reduce_arg(x, axis, preserve_axes, "max")
def argmin(x, axis, preserve_axes=False): return reduce_arg(x, axis, preserve_axes, "min")


# ----------------------------------------------------------------------------- GEMM (ops/gemm.rs)
def gemm(x1, x2, t1=False, t2=False):
    """gemm.rs:106-140."""
    x1, x2 = into_var(x1).organize(), into_var(x2).organize()
    if x1.dtype != x2.dtype:
        raise abi.DTypeError(abi.ERR_DTYPE, "gemm operands differ in dtype (gemm.rs:113)")
    if x1.rank != 2 or x2.rank != 2:
        raise abi.ShapeError(abi.ERR_SHAPE, "gemm needs rank-2 operands")
    e1, e2 = x1.extents, x2.extents
    h, c1 = (e1[1], e1[0]) if t1 else (e1[0], e1[1])
    w, c2 = (e2[0], e2[1]) if t2 else (e2[1], e2[0])
    if c1 != c2:
        raise abi.ShapeError(abi.ERR_SHAPE, f"gemm inner dimensions {c1} and {c2} differ (gemm.rs:124)")
    return Var(Shape([h, w]), x1.dtype, "gemm", [x1, x2], {"ta": bool(t1), "tb": bool(t2)})


def gemm_batched(x1, x2, t1=False, t2=False):
    """gemm.rs:253-290."""
    x1, x2 = into_var(x1).organize(), into_var(x2).organize()
    if x1.rank != 3 or x2.rank != 3 or x1.extents[0] != x2.extents[0]:
        raise abi.ShapeError(abi.ERR_SHAPE, "gemm_batched: batch extents differ (gemm.rs:261)")
    if x1.dtype != x2.dtype:
        raise abi.DTypeError(abi.ERR_DTYPE, "gemm_batched operands differ in dtype (gemm.rs:262)")
    e1, e2 = x1.extents[1:], x2.extents[1:]
    h, c1 = (e1[1], e1[0]) if t1 else (e1[0], e1[1])
    w, c2 = (e2[0], e2[1]) if t2 else (e2[1], e2[0])
    if c1 != c2:
        raise abi.ShapeError(abi.ERR_SHAPE, "gemm_batched inner dimensions differ (gemm.rs:276)")
    return Var(Shape([x1.extents[0], h, w]), x1.dtype, "gemm_batched", [x1, x2], {"ta": bool(t1), "tb": bool(t2)})


def matmul(x1, x2):
    """gemm.rs:30-51."""
    x1, x2 = into_var(x1), into_var(x2)
    ext = x1.extents[:-1] + x2.extents[1:]
    a = x1.view([x1.size() // x1.extents[-1], x1.extents[-1]])
    b = x2.view([x2.extents[0], x2.size() // x2.extents[0]])
    return gemm(a, b).view(ext)


def matmul_batched(x1, x2):
    """gemm.rs:53-104.  When both operands have the same rank (<= 4) and every leading axis is a
    batch axis, the product is expressed on the strided operands directly ("matmul_nd"), which the
    backend runs without the reference's organize() copies; otherwise the reference's own
    view -> gemm_batched -> view composition is used."""
    x1, x2 = into_var(x1), into_var(x2)
    batch = []
    for i in range(min(x1.rank - 2, x2.rank - 2)):
        if x1.extents[i] == x2.extents[i]:
            batch.append(x1.extents[i])
        else:
            break
    bl = len(batch)
    if bl == 0:
        raise abi.ShapeError(abi.ERR_SHAPE, "batch dim incorrect!")
    bs = 1
    for b in batch:
        bs *= b
    ext = batch + x1.extents[bl:x1.rank - 1] + x2.extents[bl + 1:]
    if (_FUSION["on"] and x1.rank == x2.rank and x1.rank <= 4 and bl == x1.rank - 2
            and x1.extents[-1] == x2.extents[-2] and x1.dtype == x2.dtype == FLOAT):
        return Var(Shape(ext), x1.dtype, "matmul_nd", [x1, x2])
    a = x1.view([bs, x1.size() // (x1.extents[-1] * bs), x1.extents[-1]])
    b = x2.view([bs, x2.extents[bl], x2.size() // (x2.extents[bl] * bs)])
    return gemm_batched(a, b).view(ext)


def matmul_batched_composed(x1, x2):
    """matmul_batched exactly as the reference composes it (view -> gemm_batched -> view), whatever
    the fusion setting; the gradient of the strided form is taken through this."""
    on = _FUSION["on"]
    _FUSION["on"] = False
    try:
        return matmul_batched(x1, x2)
    finally:
        _FUSION["on"] = on


# ----------------------------------------------------------------------------- random fills (ops/rand.rs)
def uniform(extents, seed=None):
    """rand.rs:20-28.  The reference draws two 32-bit seeds from the host RNG at every evaluation
    (rand.rs:70); `seed=(x, y)` fixes them, None draws them when the node is evaluated."""
    if isinstance(extents, int):
        extents = [extents]
    return Var(Shape(list(extents)), FLOAT, "rand_uniform", attrs={"seed": tuple(seed) if seed is not None else None})


def normal(extents, seed=None):
    """rand.rs:30-37 (Box-Muller on xorshift128 samples)."""
    if isinstance(extents, int):
        extents = [extents]
    return Var(Shape(list(extents)), FLOAT, "rand_normal", attrs={"seed": tuple(seed) if seed is not None else None})


# ----------------------------------------------------------------------------- conv (ops/conv.rs)
def _pair(v):
    return [int(v), int(v)] if isinstance(v, (int, np.integer)) else [int(v[0]), int(v[1])]


def conv_size(size, ker, stride, pad, dil):
    """conv.rs:47-59."""
    return [(size[i] + 2 * pad[i] - dil[i] * (ker[i] - 1) - 1) // stride[i] + 1 for i in range(2)]


def im2col(x, ker_size, stride, padding, dilation):
    """conv.rs:188-226.  Every pair is [w, h]."""
    x = into_var(x).organize()
    ker, stride, pad, dil = _pair(ker_size), _pair(stride), _pair(padding), _pair(dilation)
    if x.rank != 4:
        raise abi.ShapeError(abi.ERR_SHAPE, "im2col needs [N,H,W,C] (conv.rs:199)")
    n, h, w, c = x.extents
    col = conv_size([w, h], ker, stride, pad, dil)
    return Var(Shape([n, col[1], col[0], ker[1], ker[0], c]), x.dtype, "im2col", [x],
               {"ker": ker, "stride": stride, "pad": pad, "dil": dil})


def col2im(x, img_size, ker_size, stride, padding, dilation):
    """conv.rs:229-264.  img_size and every pair are [w, h]; x is [N,OH,OW,KH,KW,C]."""
    x = into_var(x).organize()
    ker, stride, pad, dil = _pair(ker_size), _pair(stride), _pair(padding), _pair(dilation)
    if x.rank != 6:
        raise abi.ShapeError(abi.ERR_SHAPE, "col2im needs [N,OH,OW,KH,KW,C] (conv.rs:243)")
    return Var(Shape([x.extents[0], img_size[1], img_size[0], x.extents[5]]), x.dtype, "col2im", [x],
               {"img": list(img_size), "ker": ker, "stride": stride, "pad": pad, "dil": dil})


def conv_2d(x, filt, stride, padding, dilation):
    """conv.rs:61-96: filter [KH,KW,C,OC]."""
    filt = into_var(filt)
    if filt.rank != 4:
        raise abi.ShapeError(abi.ERR_SHAPE, "conv_2d filter must be [KH,KW,C,OC] (conv.rs:70)")
    kh, kw, cin, cout = filt.extents
    col = im2col(x, [kw, kh], stride, padding, dilation)
    if col.extents[5] != cin:
        raise abi.ShapeError(abi.ERR_SHAPE, "conv_2d channel mismatch (conv.rs:86)")
    n, ch, cw = col.extents[:3]
    col = col.view([n * ch * cw, kh * kw * cin])
    f = filt.view([kh * kw * cin, cout])
    return col.matmul(f).view([n, ch, cw, cout])


def conv_transpose_2d(x, filt, stride, padding, dilation):
    """conv.rs:98-140, as written there: the filter's axis 2 is taken as the output channel count and its
    permutation (2,0,1,3) is viewed as [C_in, KH*KW*that], so extent 3 must equal x's channels; the product's
    [N,H,W,KH,KW,OC] columns are folded by col2im onto an image of (size-1)*stride - 2*pad + dil*(ker-1)
    per side (conv.rs:33-45: one less than the usual transposed-convolution size)."""
    filt, x = into_var(filt), into_var(x)
    if filt.rank != 4 or x.rank != 4:
        raise abi.ShapeError(abi.ERR_SHAPE, "conv_transpose_2d needs x [N,H,W,C] and a rank-4 filter (conv.rs:104-116)")
    n, h, w, cin = x.extents
    kh, kw, cout = filt.extents[0], filt.extents[1], filt.extents[2]
    ker, stride, pad, dil = [kw, kh], _pair(stride), _pair(padding), _pair(dilation)
    if filt.extents[3] != cin:
        raise abi.ShapeError(abi.ERR_SHAPE, "conv_transpose_2d: filter does not view as [C_in, KH*KW*OC] (conv.rs:125)")
    f = filt.permute([2, 0, 1, 3]).organize().view([cin, kh * kw * cout])
    col = x.view([n * h * w, cin]).matmul(f).view([n, h, w, kh, kw, cout])
    out = [(s - 1) * st - 2 * p + d * (k - 1) for s, k, st, p, d in zip([w, h], ker, stride, pad, dil)]
    if min(out) < 1:
        raise abi.ShapeError(abi.ERR_SHAPE, "conv_transpose_2d: empty output (conv.rs:42)")
    return col2im(col, out, ker, stride, pad, dil)


def avg_pool_2d(x, ker_size, stride, padding, dilation):
    """conv.rs:143-153."""
    return im2col(x, ker_size, stride, padding, dilation).mean([3, 4], False)


def max_pool_2d(x, ker_size, stride, padding, dilation):
    """conv.rs:155-165."""
    return im2col(x, ker_size, stride, padding, dilation).max([3, 4], False)


def batch_norm_2d(x, gamma, beta, mean_, var_, eps):
    """conv.rs:167-185."""
    x = into_var(x)
    xc = (x - mean_) / (into_var(var_) + float(eps)).sqrt()
    return into_var(gamma) * xc + beta


# ----------------------------------------------------------------------------- evaluation
def _lit_bits(value, dtype):
    np_t = {FLOAT: np.float32, INT: np.int32, UINT: np.uint32}[dtype]
    return int(np.array(value).astype(np_t).view(np.uint32))


class _MapBuilder:
    """Collects one fused map: prefix program + deduplicated input tensors."""

    def __init__(self):
        self.prog = []
        self.leaves = []   # Tensors
        self.keys = {}

    def leaf(self, t):
        key = (t.buf.ptr, tuple(t.shape.extents), tuple(t.shape.strides), t.shape.offset, t.dtype)
        if key not in self.keys:
            self.keys[key] = len(self.leaves)
            self.leaves.append(t)
        self.prog.append((abi.EXPR_INPUT, self.keys[key], 0, 0))


def fresh_seed():
    """Two 32-bit seeds from the host's entropy, as the reference draws them per call (rand.rs:70, 113)."""
    return tuple(int(b) for b in np.frombuffer(os.urandom(8), np.uint32))


def refresh_derived(ctx, entries):
    """Re-run the calls that build cached derived data when parameters changed since they last ran."""
    for e in entries:
        if e["epoch"] != _PARAM_EPOCH[0]:
            for fn, args, _ in e["calls"]:
                ctx.check(fn(ctx.handle, *args))
            e["epoch"] = _PARAM_EPOCH[0]


def evaluate_fresh(ctx, targets):
    """Evaluate `targets` without keeping their tensors on the Vars (the reference clears ctx.data
    between evaluations for the same effect, var.rs:121)."""
    ev = _Evaluator(ctx, targets)
    return [ev.get(t) for t in targets]


def evaluate(ctx, targets):
    """Context::eval (context.rs:96-117): evaluate `targets`, keep their tensors on the Vars."""
    ev = _Evaluator(ctx, targets)
    out = [ev.get(t) for t in targets]
    for t, v in zip(targets, out):
        t.value = v
    return out


class Program:
    """Program::compile / Program::exec (session.rs:62-206, 208-468) for a fixed graph: the first
    evaluation decides every launch (fusion, epilogues, layouts) and allocates every intermediate;
    `run()` replays exactly those launches on the same buffers, so a repeated forward pass costs no
    graph walking and no allocation.  New input values are supplied by writing into the data
    tensors the graph was built on (`Tensor.copy_from_numpy`)."""

    def __init__(self, ctx, targets):
        self.ctx = ctx
        self.calls = []
        self.graph = None
        self.targets = list(targets)
        self._ev = _Evaluator(ctx, targets, record=self.calls)
        self.outputs = [self._ev.get(t) for t in targets]
        self.derived = self._ev.derived
        self.reseed = self._ev.reseed
        self.changes_params = False  # set by optimizers: every run rewrites parameter values

    def bind(self):
        """Keep each target's output tensor on its Var (the role of ctx.data after Program::exec,
        session.rs:657-664): later expressions, e.g. an optimizer's, can then use the targets as data.
        The tensors are rewritten in place by every run."""
        for t, o in zip(self.targets, self.outputs):
            t.value = o
        return self

    def run_eager(self):
        h, check = self.ctx.handle, self.ctx.check
        refresh_derived(self.ctx, self.derived)
        if self.changes_params:
            params_changed()
        for sx, sy in self.reseed:  # unseeded random fills draw new seeds at every evaluation
            sx.value, sy.value = fresh_seed()
        for fn, args, _ in self.calls:
            rc = fn(h, *args)
            if rc:
                check(rc)
        self.ctx.launches += len(self.calls)
        return self.outputs

    def capture(self):
        """Record the launch sequence into a HIP graph (sg_graph_begin/end); `run()` then replays it with
        one submission instead of one host call per operator.  The sequence has already run once in
        the constructor, so every expression kernel is built and every buffer exists."""
        if self.graph is not None:
            return self
        if self.reseed:
            raise ValueError("a program with unseeded random fills cannot be captured: a graph replays fixed kernel "
                             "arguments, so every replay would repeat the same random numbers (give the nodes seeds)")
        lib, h = self.ctx._lib, self.ctx.handle
        self.ctx.check(lib.sg_graph_begin(h))
        rc_call = 0
        for fn, args, _ in self.calls:
            rc_call = fn(h, *args)
            if rc_call:
                break
        g = C.c_void_p()
        rc_end = lib.sg_graph_end(h, C.byref(g))
        if rc_call:
            if not rc_end:
                lib.sg_graph_destroy(h, g)
            self.ctx.check(rc_call)
        self.ctx.check(rc_end)
        self.graph = g
        return self

    def release_graph(self):
        if self.graph is not None and self.ctx.handle:
            self.ctx._lib.sg_graph_destroy(self.ctx.handle, self.graph)
        self.graph = None

    def run(self):
        if self.graph is None:
            return self.run_eager()
        refresh_derived(self.ctx, self.derived)
        if self.changes_params:
            params_changed()
        self.ctx.check(self.ctx._lib.sg_graph_launch(self.ctx.handle, self.graph))
        self.ctx.launches += 1
        return self.outputs


def _allow_depth(targets):
    """The evaluator walks the graph recursively, a handful of Python frames per node: raise the
    interpreter's recursion limit to fit the deepest chain of this graph (MobileNetV2 is ~400 nodes deep)."""
    import sys
    depth, memo = 0, {}
    for t in targets:
        stack = [t]
        while stack:
            n = stack[-1]
            if id(n) in memo:
                stack.pop()
                continue
            todo = [i for i in n.inputs if id(i) not in memo] if n.value is None else []
            if todo:
                stack.extend(todo)
                continue
            memo[id(n)] = 1 + max((memo[id(i)] for i in n.inputs), default=0) if n.value is None else 0
            stack.pop()
        depth = max(depth, memo[id(t)])
    need = min(12 * depth + 1000, 60000)
    if sys.getrecursionlimit() < need:
        sys.setrecursionlimit(need)


def _category(v):
    """Operator::cat (ops.rs:219-227): maps, Expand (the only Layout, core.rs:319-321), Gemm/GemmBatched
    (Contract, gemm.rs:166, 328), reduce (reduce.rs:327); everything else keeps the trait default, Other
    (ops.rs:86-88).  The fused nodes this front-end adds stand for chains containing reductions or products."""
    if v.op in MAP_OPS:
        return "map"
    if v.op == "expand":
        return "layout"
    if v.op in GEMM_OPS:
        return "contract"
    if v.op == "reduce":
        return "reduce"
    return "other"


def state_partition(targets, inputs=(), decide_only=False):
    """Phase 1 of Program::compile (session.rs:101-169): which nodes are STATES, i.e. evaluated once and
    retained; every other node is recomputed inside each routine that needs it.  Candidates are the operator
    nodes with two or more consumers plus the outputs, visited in topological order; a candidate's ancestry
    is walked up to data, earlier states and the program inputs, counting every visited node (a node reached
    twice counts twice: the walk is over the expanded tree) and collecting the distinct leaves.  It is a state
    if it is an output, if a Contract / Reduce / Other operator lies on the way, or if nodes x leaves > THRES.
    Returns {id(state): set of ids of its routine's inputs}; with decide_only the walk stops as soon as the
    answer is known and the input sets are left incomplete."""
    targets = list(targets)
    input_ids = {id(v) for v in inputs}
    target_ids = {id(t) for t in targets}

    def is_op(v):
        return v.value is None and v.op != "data"

    nodes, order, stack = {}, {}, [(t, False) for t in targets]
    while stack:  # reachable nodes and their depth (a topological order)
        v, expanded = stack.pop()
        if expanded:
            order[id(v)] = 1 + max((order[id(i)] for i in v.inputs), default=0) if is_op(v) and id(v) not in input_ids else 0
            continue
        if id(v) in nodes:
            continue
        nodes[id(v)] = v
        stack.append((v, True))
        if is_op(v) and id(v) not in input_ids:
            stack.extend((i, False) for i in v.inputs)
    edges = {}
    for v in nodes.values():
        if is_op(v) and id(v) not in input_ids:
            for i in v.inputs:
                edges[id(i)] = edges.get(id(i), 0) + 1
    cand = [nodes[k] for k, n in edges.items() if n >= 2 and is_op(nodes[k]) and k not in input_ids and k not in target_ids]
    cand += targets
    cand.sort(key=lambda v: order[id(v)])
    states = {}
    for node in cand:
        if id(node) in states:
            continue
        leaves, num_ops, complex_op, stack = set(), 0, False, [node]
        is_target = id(node) in target_ids
        while stack:
            v = stack.pop()
            num_ops += 1
            if not is_op(v) or id(v) in states or id(v) in input_ids:
                leaves.add(id(v))
            else:
                stack.extend(v.inputs)
                if _category(v) in ("contract", "reduce", "other"):
                    complex_op = True
            if decide_only and (is_target or complex_op or (leaves and num_ops > THRES)):
                break
        if is_target or complex_op or num_ops * len(leaves) > THRES:
            states[id(node)] = leaves
    return states


def _merge_common_subgraphs(targets):
    """Structurally identical operations on the same inputs are computed once: inputs of every node are
    re-pointed at the first node seen with the same (operator, attributes, inputs).  BERT rebuilds the
    extended attention mask in each of its layers (bert.rs:264-268, 304-314); this leaves one."""
    canon, table = {}, {}
    order, seen, stack = [], set(), [(t, False) for t in targets]
    while stack:
        v, expanded = stack.pop()
        if expanded:
            order.append(v)
            continue
        if id(v) in seen:
            continue
        seen.add(id(v))
        stack.append((v, True))
        if v.value is None:
            for i in v.inputs:
                stack.append((i, False))
    for v in order:
        if v.value is not None or v.op == "data":
            canon[id(v)] = v
            continue
        v.inputs = tuple(canon[id(i)] for i in v.inputs)
        key = (v.op, v.dtype, tuple(v.shape.extents), tuple(v.shape.strides), v.shape.offset,
               repr(sorted(v.attrs.items(), key=lambda kv: kv[0])), tuple(id(i) for i in v.inputs))
        if v.op in ("rand_uniform", "rand_normal") and v.attrs.get("seed") is None:
            key += (id(v),)  # every unseeded node is its own draw (rand.rs:70, 113): never merged
        canon[id(v)] = table.setdefault(key, v)


def _is_relu_mask(m):
    """m = float(x > 0), the factor of nn.rs:33-40; returns x or None."""
    if m.value is not None or m.op != "unary" or m.attrs.get("name") != "cast_float":
        return None
    g = m.inputs[0]
    if g.value is not None or g.op != "binary" or g.attrs.get("name") != "gt":
        return None
    z = g.inputs[1]
    if z.value is None and z.op == "literal" and z.attrs.get("value") == 0.0 and z.dtype == FLOAT:
        return g.inputs[0]
    return None


def _relu_masks_from_outputs(targets):
    """Where y = float(x > 0) * x (relu, nn.rs:33-40) and the same factor float(x > 0) is also used elsewhere (the
    backward pass multiplies the incoming gradient by it, map.rs:1014-1041), those other uses read float(y > 0)
    instead: y > 0 exactly when x > 0 (y is x or 0; a NaN fails both tests), so no value changes, and x, left
    with relu as its only consumer, can be folded into the product that makes it instead of being stored."""
    order, seen, stack = [], set(), [(t, False) for t in targets]
    while stack:
        v, expanded = stack.pop()
        if expanded:
            order.append(v)
            continue
        if id(v) in seen:
            continue
        seen.add(id(v))
        stack.append((v, True))
        if v.value is None:
            for i in v.inputs:
                stack.append((i, False))
    relu_of = {}  # id(mask node) -> (mask node, relu node)
    for y in order:
        if y.value is None and y.op == "binary" and y.attrs.get("name") == "mul":
            for m, x in ((y.inputs[0], y.inputs[1]), (y.inputs[1], y.inputs[0])):
                if _is_relu_mask(m) is x and id(m) not in relu_of:
                    relu_of[id(m)] = (m, y)
    if not relu_of:
        return
    from_output = {}
    for v in order:
        if v.value is not None or not any(id(i) in relu_of for i in v.inputs):
            continue
        new = []
        for i in v.inputs:
            hit = relu_of.get(id(i))
            if hit is None or hit[1] is v:
                new.append(i)
                continue
            y = hit[1]
            if id(y) not in from_output:
                from_output[id(y)] = binary_map(y, 0.0, "gt").float()
            new.append(from_output[id(y)])
        v.inputs = tuple(new)


class _Evaluator:
    def __init__(self, ctx, targets, record=None):
        self.ctx = ctx
        self.lib = ctx._lib
        self.memo = {}
        self.users = {}
        self.targets = {id(t) for t in targets}
        if _FUSION["on"]:
            _merge_common_subgraphs(targets)
            _relu_masks_from_outputs(targets)
        # which shared nodes are stored once and which are recomputed in every consumer (session.rs:101-169)
        self.states = state_partition(targets, decide_only=True) if _FUSION["on"] else {}
        _allow_depth(targets)
        seen = set()
        stack = list(targets)
        while stack:
            v = stack.pop()
            if id(v) in seen:
                continue
            seen.add(id(v))
            if v.value is not None:
                continue
            for i in v.inputs:
                self.users.setdefault(id(i), []).append(v)
                stack.append(i)
        self.keep = {}  # id -> Var, keeps nodes alive while ids are used as keys
        self.record = record
        self.keepalive = []
        # Memory behaviour of Program::exec (session.rs:208-330) for a one-off evaluation: intermediates
        # are dropped once every consumer has run, and when an allocation runs out of memory the cheapest
        # retained intermediate (recompute time per byte) is dropped and recomputed on demand later.  A
        # recorded Program keeps every buffer instead: its launches are replayed on them.
        self.derived = []  # cached derived-data entries this evaluation relies on (see refresh_derived)
        self.reseed = []   # seed arguments of unseeded random fills (drawn per evaluation, rand.rs:70, 113)
        self.release = record is None
        self.computed = set()
        self.evictions = 0
        self.eviction_log = []  # one list of evicted tensor sizes (elements) per out-of-memory event, in eviction order
        self.exec_time = {}

    # ---- helpers
    def n_users(self, v):
        return len(self.users.get(id(v), ()))

    def done(self, v):
        return v.value is not None or id(v) in self.memo

    def get(self, v):
        if v.value is not None:
            return v.value
        t = self.memo.get(id(v))
        if t is None:
            if v.op == "data":
                raise RuntimeError("cannot evaluate empty var")
            t0 = time.perf_counter()
            t = getattr(self, "_ev_" + v.op)(v)
            # Routine::exec_time (session.rs:619, 667-668): host seconds spent issuing the node (and whatever it had to
            # evaluate first), the figure the eviction rule below reads
            self.exec_time[id(v)] = time.perf_counter() - t0
            self.memo[id(v)] = t
            self.keep[id(v)] = v
            self.computed.add(id(v))
            if self.release:
                self._release_consumed(v)
        return t

    def _finished(self, u, cache):
        """Every path from u to a target passes through a node that has been computed."""
        k = id(u)
        if k in self.computed or k in self.memo or u.value is not None:
            return True
        if k in self.targets:
            return False
        if k not in cache:
            cache[k] = False
            us = self.users.get(k, ())
            cache[k] = bool(us) and all(self._finished(w, cache) for w in us)
        return cache[k]

    def _release_consumed(self, v):
        """Drop the tensors that the evaluation of v consumed and nobody else still needs: the retained
        nodes reachable from v through nodes that were fused away rather than materialised."""
        cache, seen, stack = {}, set(), list(v.inputs)
        while stack:
            n = stack.pop()
            if id(n) in seen or n.value is not None:
                continue
            seen.add(id(n))
            if id(n) in self.memo:
                if id(n) not in self.targets and all(self._finished(u, cache) for u in self.users.get(id(n), ())):
                    del self.memo[id(n)]
            else:
                stack.extend(n.inputs)

    def _evict(self, needed):
        """session.rs:259-325: free at least `needed` bytes by dropping retained intermediates in the reference's
        order: smallest (exec_time + 1.0) / (size + 1.0) first (session.rs:300-310), exec_time being the host
        seconds measured when the node was evaluated.  (Issuing a node takes well under a second, so the rule
        amounts to "largest tensor first", as it does in the reference; ties there fall to a hash map's iteration
        order, here to evaluation order.)  Tensors still referenced by the operator being evaluated stay alive
        whatever is dropped here (the reference's `lock` set plays that role)."""
        start = self.ctx.mem_stats()["used"]
        cands = [self.keep[k] for k in self.memo if k not in self.targets and k in self.keep and self.keep[k].value is None
                 and self.keep[k].op != "data"]
        cands.sort(key=lambda n: (self.exec_time.get(id(n), 0.0) + 1.0) / (n.size() + 1.0))
        self.eviction_log.append([])
        for n in cands:
            del self.memo[id(n)]
            self.computed.discard(id(n))
            self.evictions += 1
            self.eviction_log[-1].append(n.size())
            if start - self.ctx.mem_stats()["used"] >= needed:
                return True
        if start - self.ctx.mem_stats()["used"] >= needed:
            return True
        self.ctx.__dict__.get("_wide_weights", {}).clear()  # rebuilt on demand; recorded Programs keep their own
        return start - self.ctx.mem_stats()["used"] >= needed

    def call(self, fn, *args):
        """Issue one operator launch through the C ABI; remember it when a Program is being compiled.
        The epilogue struct keeps pointers into `keepalive` objects, so those are stored too."""
        self.ctx.launches += 1
        while True:
            try:
                self.ctx.check(fn(self.ctx.handle, *args))
                break
            except abi.OutOfMemory as e:  # a workspace inside the library did not fit
                if not self.release or not self._evict(e.needed or 1):
                    raise
        if self.record is not None:
            self.record.append((fn, args, list(self.keepalive)))
        self.keepalive = []

    def out(self, extents, dtype):
        while True:
            try:
                return Tensor.uninit(self.ctx, extents, dtype)
            except abi.OutOfMemory as e:
                if not self.release or not self._evict(e.needed or 1):
                    raise

    # ---- layout operators: descriptor rewrites on the evaluated tensor
    def _ev_reshape(self, v):
        x = self.get(v.inputs[0])
        if not x.is_dense():
            # a strided tensor (e.g. a column block of a wider GEMM result) can often be re-viewed
            # in place; only layouts that really need it are copied (core.rs:213-233 always copies)
            sh = x.shape.reshape_view(v.extents) if _FUSION["on"] else None
            if sh is not None:
                return x.with_shape(sh)
            x = self.run_copy(x)
        return x.with_shape(Shape(v.extents, default_strides(v.extents), x.shape.offset))

    def _ev_expand(self, v):
        x = self.get(v.inputs[0])
        return x.with_shape(x.shape.expand(v.extents))

    def _ev_permute(self, v):
        x = self.get(v.inputs[0])
        return x.with_shape(x.shape.permute(v.attrs["axes"]))

    def _ev_squeeze(self, v):
        x = self.get(v.inputs[0])
        return x.with_shape(x.shape.remove(v.attrs["axis"]))

    def _ev_unsqueeze(self, v):
        x = self.get(v.inputs[0])
        return x.with_shape(x.shape.insert(v.attrs["axis"]))

    def _ev_slice(self, v):
        x = self.get(v.inputs[0])
        a = v.attrs
        return x.with_shape(x.shape.select_range(a["start"], a["end"] - 1, a["axis"]))

    # ---- maps
    def inline_ok(self, c):
        """A map operand is computed inside its consumer's kernel (Operator::fuse, ops.rs:104-161) when the
        consumer is its only one, or when the reference would not retain it either: a shared node that is no
        state is recomputed by every routine that reaches it (session.rs:157-169, 524-535)."""
        if not _FUSION["on"] or c.op not in MAP_OPS or self.done(c) or id(c) in self.targets:
            return False
        return self.n_users(c) <= 1 or id(c) not in self.states

    def inline_size(self, v, cap):
        """Program elements v would add if it and everything below it were inlined (capped)."""
        n, stack = 0, [v]
        while stack and n <= cap:
            c = stack.pop()
            n += 1
            if c.op in MAP_OPS and not self.done(c):
                stack.extend(c.inputs)
        return n

    def build_map(self, v, mb, budget):
        """Append v's expression (prefix order) to mb, inlining fusable children."""
        if v.op == "literal":
            mb.prog.append((abi.EXPR_LITERAL, 0, v.dtype, _lit_bits(v.attrs["value"], v.dtype)))
            return
        if v.op == "unary":
            mb.prog.append((abi.EXPR_UNARY, abi.U[v.attrs["name"]], 0, 0))
        elif v.op == "binary":
            mb.prog.append((abi.EXPR_BINARY, abi.B[v.attrs["name"]], 0, 0))
        else:
            mb.prog.append((abi.EXPR_TERNARY, 0, 0, 0))
        for c in v.inputs:
            room = len(mb.leaves) < abi.MAX_MAP_INPUTS - 3 and len(mb.prog) + self.inline_size(c, budget) < budget - 4
            if room and self.inline_ok(c):
                self.build_map(c, mb, budget)
            else:
                mb.leaf(self.get(c))

    def run_map(self, prog, leaves, extents, dtype):
        y = self.out(extents, dtype)
        n = len(prog)
        arr = (abi.sg_expr * n)()
        for i, (k, o, d, b) in enumerate(prog):
            arr[i].kind, arr[i].op, arr[i].dtype, arr[i].bits = k, o, d, b
        ins = (abi.sg_tensor * max(1, len(leaves)))(*[t.c() for t in leaves])
        yc = y.c()
        self.call(self.lib.sg_map, arr, n, ins, len(leaves), C.byref(yc))
        return y

    def run_copy(self, x):
        """UnaryMap::Copy as Var::organize (var.rs:506-512)."""
        return self.run_map([(abi.EXPR_UNARY, abi.U["copy"], 0, 0), (abi.EXPR_INPUT, 0, 0, 0)], [x], x.extents, x.dtype)

    def _ev_map(self, v):
        if _FUSION["on"]:
            t = self.try_gemm_chain(v)
            if t is not None:
                return t
            if v.op == "unary" and v.attrs["name"] == "copy":
                t = self.try_permuted_matmul(v)
                if t is not None:
                    return t
        mb = _MapBuilder()
        self.build_map(v, mb, abi.MAX_EXPR)
        return self.run_map(mb.prog, mb.leaves, v.extents, v.dtype)

    _ev_literal = _ev_unary = _ev_binary = _ev_cond = _ev_map

    # ---- reductions and indexing
    def _ev_reduce(self, v):
        col = v.inputs[0]
        if (_FUSION["on"] and col.op == "im2col" and self._private(col) and list(v.attrs["axes"]) == [3, 4]  # ky innermost, the kernel's order
                and v.dtype == FLOAT and os.environ.get("SAGE_FUSE_CONV", "1") != "0"):
            # max_pool_2d / avg_pool_2d (conv.rs:143-165): the window is reduced while it is read, no column tensor
            x = self.get(col.inputs[0])
            if not x.is_dense():
                x = self.run_copy(x)
            n, oh, ow, _, _, c = col.extents
            y = self.out(v.extents, FLOAT)
            a = col.attrs
            arr = lambda p: (C.c_int32 * 2)(*p)
            op = {"sum": abi.R_SUM, "prod": abi.R_PROD, "max": abi.R_MAX, "min": abi.R_MIN}[v.attrs["op"]]
            init = abi.INIT_REF_ZERO if v.attrs["init"] == "ref_zero" else abi.INIT_IDENTITY
            xc, yc = x.c(), y.with_shape(Shape([n, oh, ow, c])).c()
            self.call(self.lib.sg_pool2d, op, init, C.byref(xc), C.byref(yc), arr(a["ker"]), arr(a["stride"]), arr(a["pad"]), arr(a["dil"]))
            return y
        x = self.get(v.inputs[0])
        y = self.out(v.extents, v.dtype)
        axes = v.attrs["axes"]
        ax = (C.c_int32 * max(1, len(axes)))(*axes)
        op = {"sum": abi.R_SUM, "prod": abi.R_PROD, "max": abi.R_MAX, "min": abi.R_MIN}[v.attrs["op"]]
        init = abi.INIT_REF_ZERO if v.attrs["init"] == "ref_zero" else abi.INIT_IDENTITY
        xc, yc = x.c(), y.c()
        self.call(self.lib.sg_reduce, op, ax, len(axes), init, C.byref(xc), C.byref(yc))
        return y

    def _ev_reduce_arg(self, v):
        x = self.get(v.inputs[0])
        y = self.out(v.extents, UINT)
        xc, yc = x.c(), y.c()
        op = abi.RA_MAX if v.attrs["op"] == "max" else abi.RA_MIN
        self.call(self.lib.sg_reduce_arg, op, v.attrs["axis"], C.byref(xc), C.byref(yc))
        return y

    def _ev_gather(self, v):
        x, ind = self.get(v.inputs[0]), self.get(v.inputs[1])
        y = self.out(v.extents, v.dtype)
        xc, ic, yc = x.c(), ind.c(), y.c()
        self.call(self.lib.sg_gather, v.attrs["axis"], C.byref(xc), C.byref(ic), C.byref(yc))
        return y

    def _ev_scatter(self, v):
        x, ind = self.get(v.inputs[0]), self.get(v.inputs[1])
        y = self.out(v.extents, v.dtype)
        xc, ic, yc = x.c(), ind.c(), y.c()
        self.call(self.lib.sg_scatter, v.attrs["axis"], C.byref(xc), C.byref(ic), C.byref(yc))
        return y

    def _ev_unslice(self, v):
        x = self.get(v.inputs[0])
        y = self.out(v.extents, v.dtype)
        xc, yc = x.c(), y.c()
        self.call(self.lib.sg_unslice, v.attrs["axis"], v.attrs["start"], C.byref(xc), C.byref(yc))
        return y

    def _ev_concat(self, v):
        xs = [self.get(i) for i in v.inputs]
        y = self.out(v.extents, v.dtype)
        ins = (abi.sg_tensor * len(xs))(*[t.c() for t in xs])
        yc = y.c()
        self.call(self.lib.sg_concat, v.attrs["axis"], ins, len(xs), C.byref(yc))
        return y

    def _ev_im2col(self, v):
        x = self.get(v.inputs[0])
        if not x.is_dense():
            x = self.run_copy(x)
        y = self.out(v.extents, v.dtype)
        a = v.attrs
        arr = lambda p: (C.c_int32 * 2)(*p)
        xc, yc = x.c(), y.c()
        self.call(self.lib.sg_im2col, C.byref(xc), C.byref(yc), arr(a["ker"]), arr(a["stride"]), arr(a["pad"]), arr(a["dil"]))
        return y

    def _ev_rand(self, v):
        seed = v.attrs["seed"]
        fresh = seed is None
        if fresh:
            seed = fresh_seed()
        y = self.out(v.extents, FLOAT)
        yc = y.c()
        fn = self.lib.sg_rand_uniform if v.op == "rand_uniform" else self.lib.sg_rand_normal
        sx, sy = C.c_uint32(seed[0] & 0xFFFFFFFF), C.c_uint32(seed[1] & 0xFFFFFFFF)
        self.call(fn, sx, sy, C.byref(yc))
        if fresh:
            self.reseed.append((sx, sy))  # a recorded Program redraws these before every replay
        return y

    _ev_rand_uniform = _ev_rand_normal = _ev_rand

    def _ev_col2im(self, v):
        x = self.get(v.inputs[0])
        if not x.is_dense():
            x = self.run_copy(x)
        y = self.out(v.extents, v.dtype)
        a = v.attrs
        arr = lambda p: (C.c_int32 * 2)(*p)
        xc, yc = x.c(), y.c()
        self.call(self.lib.sg_col2im, C.byref(xc), C.byref(yc), arr(a["ker"]), arr(a["stride"]), arr(a["pad"]), arr(a["dil"]))
        return y

    # ---- GEMM family, with optional epilogue and destination layout
    def _epi_struct(self, epi, keep):
        if not epi:
            return None
        e = abi.sg_gemm_epilogue()
        e.alpha = float(epi.get("alpha", 1.0))
        e.act = epi.get("act", abi.ACT_NONE)
        e.act_post = epi.get("act_post", abi.ACT_NONE)
        if epi.get("bias") is not None:
            bc = epi["bias"].c()
            keep.append(bc)
            e.bias = C.pointer(bc)
        if epi.get("res") is not None:
            rc_ = epi["res"].c()
            keep.append(rc_)
            e.residual = C.pointer(rc_)
        return e

    def run_gemm(self, g, epi=None, dest=None):
        """Run gemm / gemm_batched / matmul_nd node `g`.  `dest`: a Tensor view with g's extents to
        write into (any batch strides, unit last stride); default a fresh dense tensor."""
        if _FUSION["on"] and dest is None:
            t = self.try_conv(g, epi)
            if t is not None:
                return t
        a, b = self.get(g.inputs[0]), self.get(g.inputs[1])
        keep = self.keepalive
        e = self._epi_struct(epi, keep)
        if e is not None:
            keep.append(e)
        ep = C.byref(e) if e is not None else None
        y = dest if dest is not None else self.out(g.extents, FLOAT)
        if g.op == "matmul_nd":
            def usable(t):
                r = t.rank
                return (t.strides[r - 1] == 1 or t.strides[r - 2] == 1 or t.extents[r - 1] == 1 or t.extents[r - 2] == 1)
            if not usable(a):
                a = self.run_copy(a)
            if not usable(b):
                b = self.run_copy(b)
            ac, bc, yc = a.c(), b.c(), y.c()
            self.call(self.lib.sg_matmul_strided, C.byref(ac), C.byref(bc), C.byref(yc), ep)
            return y
        if not a.is_dense():
            a = self.run_copy(a)
        if not b.is_dense():
            b = self.run_copy(b)
        ac, bc, yc = a.c(), b.c(), y.c()
        fn = self.lib.sg_gemm if g.op == "gemm" else self.lib.sg_gemm_batched
        self.call(fn, int(g.attrs["ta"]), int(g.attrs["tb"]), C.byref(ac), C.byref(bc), C.byref(yc), ep)
        return y

    def try_conv(self, g, epi):
        """conv_2d's `view(im2col(x)) . view(filter)` (conv.rs:61-96) as one sg_conv2d launch: the column
        matrix is consumed by this product only, so it is never written."""
        if g.op != "gemm" or g.attrs["ta"] or g.attrs["tb"] or os.environ.get("SAGE_FUSE_CONV", "1") == "0":
            return None
        col = g.inputs[0]
        while col.op == "reshape" and self._private(col):
            col = col.inputs[0]
        if col.op != "im2col" or not self._private(col):
            return None
        f = g.inputs[1]
        while f.op == "reshape" and f.value is None:
            f = f.inputs[0]
        a = col.attrs
        n, oh, ow, kh, kw, c = col.extents
        if f.rank != 4 or f.extents[:3] != [kh, kw, c] or a["ker"] != [kw, kh]:
            return None
        # the product must be exactly [n*oh*ow, kh*kw*c] . [kh*kw*c, oc]: any other 2-D factorisation of the column
        # tensor or of the filter is a different contraction and runs as im2col + gemm
        if list(g.inputs[0].extents) != [n * oh * ow, kh * kw * c] or list(g.inputs[1].extents) != [kh * kw * c, f.extents[3]]:
            return None
        x, ft = self.get(col.inputs[0]), self.get(f)
        if not x.is_dense():
            x = self.run_copy(x)
        if not ft.is_dense():
            ft = self.run_copy(ft)
        keep = self.keepalive
        e = self._epi_struct(epi, keep)
        if e is not None:
            keep.append(e)
        y = self.out(g.extents, FLOAT)
        arr = lambda p: (C.c_int32 * 2)(*p)
        xc, fc = x.c(), ft.c()
        yc = y.with_shape(Shape([n, oh, ow, g.extents[1]])).c()
        self.call(self.lib.sg_conv2d, C.byref(xc), C.byref(fc), C.byref(yc), arr(a["stride"]), arr(a["pad"]), arr(a["dil"]),
                  C.byref(e) if e is not None else None)
        return y

    def _ev_gemm(self, v):
        return self.run_gemm(v)

    _ev_gemm_batched = _ev_gemm

    def _ev_matmul_nd(self, v):
        if _FUSION["on"]:
            t = self.try_attention(v, None)
            if t is not None:
                return t
        return self.run_gemm(v)

    # ---- pattern: softmax(scale * q.k^T + per-key addend) . v  (bert.rs:262-271) as one kernel
    def _private(self, v):
        """v is consumed exactly once, not yet evaluated and not asked for by the caller."""
        return not self.done(v) and self.n_users(v) == 1 and id(v) not in self.targets

    def try_attention(self, g, dest):
        pr, vv = g.inputs
        if os.environ.get("SAGE_FUSE_ATTENTION", "1") == "0":  # measurement switch: run the chain operator by operator
            return None
        if g.op != "matmul_nd" or pr.op != "softmax" or not self._private(pr) or g.rank > 4:
            return None
        x = pr.inputs[0]
        add = None
        if x.op == "binary" and x.attrs["name"] == "add" and self._private(x):
            cands = [(x.inputs[0], x.inputs[1]), (x.inputs[1], x.inputs[0])]
        else:
            cands = [(x, None)]
        for s_node, add in cands:
            chain = [x] if add is not None else []
            scale = 1.0
            inner = s_node
            if (s_node.op == "binary" and s_node.attrs["name"] in ("mul", "div") and s_node.inputs[1].op == "literal"
                    and s_node.inputs[1].dtype == FLOAT):
                lit = float(np.float32(s_node.inputs[1].attrs["value"]))
                if s_node.attrs["name"] == "div":
                    if lit == 0.0 or np.frexp(lit)[0] != 0.5:  # x/c == x*(1/c) only for powers of two
                        continue
                    lit = 1.0 / lit
                chain.append(s_node)
                scale, inner = lit, s_node.inputs[0]
            chain.append(inner)
            if inner.op != "matmul_nd" or inner.rank != g.rank or not all(self._private(n) for n in chain):
                continue
            qv, ktv = inner.inputs
            d = qv.extents[-1]
            if d not in (32, 64) or vv.extents[-1] != d or qv.dtype != FLOAT or vv.dtype != FLOAT:
                continue
            q, kt, vt = self.get(qv), self.get(ktv), self.get(vv)
            r = g.rank
            k = kt.with_shape(kt.shape.swap(r - 2, r - 1))
            if q.strides[-1] != 1 or k.strides[-1] != 1 or vt.strides[-1] != 1:
                continue
            at = None
            if add is not None:
                at = self.get(add)
                if (at.rank != r or at.extents != inner.extents or at.dtype != FLOAT
                        or (at.extents[-2] > 1 and at.strides[-2] != 0) or (at.extents[-1] > 1 and at.strides[-1] != 1)):
                    continue
            y = dest if dest is not None else self.out(g.extents, FLOAT)
            qc, kc, vc, yc = q.c(), k.c(), vt.c(), y.c()
            ac = at.c() if at is not None else None
            self.call(self.lib.sg_attention, C.byref(qc), C.byref(kc), C.byref(vc), C.byref(ac) if ac is not None else None,
                      C.c_float(scale), C.byref(yc))
            return y
        return None

    # ---- pattern: maps that directly consume a GEMM become its epilogue
    @staticmethod
    def _skip_reshape(v, chain):
        while v.op == "reshape":
            chain.append(v)
            v = v.inputs[0]
        return v

    def _match_act(self, v, chain):
        """relu(x) = float(x > 0) * x  (nn.rs:33-40);  gelu(x) = (x*0.5) * (erf(x/sqrt 2) + 1)."""
        def is_lit(n, val):
            return n.op == "literal" and n.dtype == FLOAT and abs(float(n.attrs["value"]) - val) < 1e-6 * max(1.0, abs(val))
        if v.op != "binary" or v.attrs["name"] != "mul":
            return None, v
        l, r = v.inputs
        if (l.op == "unary" and l.attrs["name"] == "cast_float" and l.inputs[0].op == "binary"
                and l.inputs[0].attrs["name"] == "gt" and l.inputs[0].inputs[0] is r and is_lit(l.inputs[0].inputs[1], 0.0)):
            chain.extend([l, l.inputs[0]])
            return abi.ACT_RELU, r
        if (l.op == "binary" and l.attrs["name"] == "mul" and is_lit(l.inputs[1], 0.5)
                and r.op == "binary" and r.attrs["name"] == "add" and is_lit(r.inputs[1], 1.0)):
            x = l.inputs[0]
            e = r.inputs[0]
            if (e.op == "unary" and e.attrs["name"] == "erf" and e.inputs[0].op == "binary" and e.inputs[0].attrs["name"] == "div"
                    and e.inputs[0].inputs[0] is x and is_lit(e.inputs[0].inputs[1], float(np.sqrt(np.float32(2.0))))):
                chain.extend([l, r, e, e.inputs[0]])
                return abi.ACT_GELU_ERF, x
        return None, v

    def _match_core(self, v, chain):
        """[reshape*] ( G | G*lit | G/2^k | (..)+bias ) -> dict(g, alpha, bias) or None."""
        v = self._skip_reshape(v, chain)
        if v.op in GEMM_OPS:
            if v.dtype != FLOAT or self.done(v):
                return None
            chain.append(v)
            return {"g": v, "alpha": 1.0, "bias": None}
        if v.op != "binary":
            return None
        name = v.attrs["name"]
        l, r = v.inputs
        if name == "add":
            for y, b in ((l, r), (r, l)):
                if b.op == "expand":
                    src = b.inputs[0]
                    n = v.extents[-1]
                    if src.size() == n and src.extents[-1] == n and b.shape.strides[-1] in (1,) and all(s == 0 for s in b.shape.strides[:-1]):
                        sub = []
                        m = self._match_scaled(y, sub)
                        if m is not None and m["g"].extents[-1] == n:
                            chain.append(v)
                            chain.extend(sub)
                            m["bias"] = src
                            return m
            return None
        return self._match_scaled(v, chain)

    def _match_scaled(self, v, chain):
        v = self._skip_reshape(v, chain)
        if v.op in GEMM_OPS:
            if v.dtype != FLOAT or self.done(v):
                return None
            chain.append(v)
            return {"g": v, "alpha": 1.0, "bias": None}
        if v.op == "binary" and v.attrs["name"] in ("mul", "div") and v.inputs[1].op == "literal" and v.inputs[1].dtype == FLOAT:
            s = float(np.float32(v.inputs[1].attrs["value"]))
            if v.attrs["name"] == "div":
                m_, e_ = np.frexp(s)
                if s == 0.0 or m_ != 0.5:  # only exact for powers of two
                    return None
                s = 1.0 / s
            sub = [v]
            g = self._skip_reshape(v.inputs[0], sub)
            if g.op in GEMM_OPS and g.dtype == FLOAT and not self.done(g):
                sub.append(g)
                chain.extend(sub)
                return {"g": g, "alpha": s, "bias": None}
        return None

    def try_gemm_chain(self, v):
        if v.op not in ("binary",):
            return None
        chain = []
        act, x = self._match_act(v, chain)
        m = None
        res = None
        if act is not None:
            chain.append(x)
            sub = []
            m = self._match_core(x, sub)
            if m is not None:
                m["act"] = act
                chain.extend(sub)
            else:
                m, res = self._match_res(x, chain)
                if m is not None:
                    m["act_post"] = act
        else:
            sub = []
            m = self._match_core(v, sub)
            if m is not None:
                chain.extend(sub)
            else:
                m, res = self._match_res(v, chain)
        if m is None:
            return None
        g = m["g"]
        if m["bias"] is None and m["alpha"] == 1.0 and res is None and "act" not in m and "act_post" not in m:
            return None
        # every intermediate node must be used only inside the pattern, or it would be computed twice
        inside = {id(n) for n in chain} | {id(v)}
        for n in chain:
            if n is v:
                continue
            if id(n) in self.targets or self.done(n):
                return None
            for u in self.users.get(id(n), ()):
                if id(u) not in inside:
                    return None
        if m["bias"] is not None and m["alpha"] == 1.0 and res is None and "act" not in m and "act_post" not in m:
            t = self.try_sibling_gemms(v, m)
            if t is not None:
                return t
        epi = {"alpha": m["alpha"], "act": m.get("act", abi.ACT_NONE), "act_post": m.get("act_post", abi.ACT_NONE)}
        if m["bias"] is not None:
            bt = self.get(m["bias"])
            if not bt.is_dense():
                return None
            epi["bias"] = bt
        if res is not None:
            rt = self.get(res)
            if not rt.is_dense():
                return None
            epi["res"] = rt.with_shape(Shape(g.extents, default_strides(g.extents), rt.shape.offset))
        y = self.run_gemm(g, epi)
        return y.with_shape(Shape(v.extents, default_strides(v.extents), y.shape.offset))

    # ---- pattern: several Dense layers reading the same activations become one wider GEMM
    def _dense_chain_above(self, g):
        """gemm node g -> the `reshape*(g) + expand(bias)` node that is its only consumer chain, or None."""
        n = g
        while True:
            us = self.users.get(id(n), ())
            if len(us) != 1 or id(n) in self.targets or self.done(n):
                return None
            u = us[0]
            if u.op == "reshape":
                n = u
                continue
            if u.op == "binary" and u.attrs["name"] == "add":
                return u
            return None

    def try_sibling_gemms(self, v, m):
        """Dense layers that share their input (the q/k/v projections, bert.rs:254-256) are the same
        A times different weight matrices: run them as ONE GEMM against the weights laid side by
        side, and hand every layer a column block of the result (a strided view, no copy).  The
        concatenated weights and biases are built once per weight set and kept on the context."""
        g = m["g"]
        if g.op != "gemm" or g.attrs["ta"] or g.attrs["tb"]:
            return None
        a_node, w_node = g.inputs
        if w_node.op == "reshape":
            w_node = w_node.inputs[0]
        if w_node.op != "data" or m["bias"].op != "data":
            return None
        root = a_node
        while root.op == "reshape":
            root = root.inputs[0]
        members = []  # (chain root node, gemm node, weight Var, bias Var)
        seen = set()
        for u1 in self.users.get(id(root), ()):
            cands = [u1] if u1.op == "gemm" else list(self.users.get(id(u1), ())) if u1.op == "reshape" else []
            for g2 in cands:
                if id(g2) in seen or g2.op != "gemm" or g2.attrs["ta"] or g2.attrs["tb"] or self.done(g2):
                    continue
                a2 = g2.inputs[0]
                r2 = a2
                while r2.op == "reshape":
                    r2 = r2.inputs[0]
                if r2 is not root or a2.extents != a_node.extents:
                    continue
                top = v if g2 is g else self._dense_chain_above(g2)
                if top is None or self.done(top):
                    continue
                sub = []
                m2 = self._match_core(top, sub)
                if m2 is None or m2["g"] is not g2 or m2["bias"] is None or m2["alpha"] != 1.0:
                    continue
                w2 = g2.inputs[1].inputs[0] if g2.inputs[1].op == "reshape" else g2.inputs[1]
                if w2.op != "data" or m2["bias"].op != "data" or w2.value is None or m2["bias"].value is None:
                    continue
                # every intermediate of the sibling must be private to its chain
                inside = {id(n) for n in sub} | {id(top)}
                if any(id(u) not in inside for n in sub if n is not top for u in self.users.get(id(n), ())):
                    continue
                seen.add(id(g2))
                members.append((top, g2, w2, m2["bias"]))
        if len(members) < 2 or not any(t is v for t, _, _, _ in members):
            return None
        members.sort(key=lambda t: id(t[2]))
        ws = [w.value for _, _, w, _ in members]
        bs = [b.value for _, _, _, b in members]
        if not all(w.is_dense() and w.rank == 2 and w.extents[0] == ws[0].extents[0] for w in ws) or not all(b.is_dense() for b in bs):
            return None
        key = tuple((w.buf.ptr, w.shape.offset, b.buf.ptr, b.shape.offset) for w, b in zip(ws, bs))
        cache = self.ctx.__dict__.setdefault("_wide_weights", {})
        if key not in cache:
            K = ws[0].extents[0]
            ntot = sum(w.extents[1] for w in ws)
            wcat, bcat = self.out([K, ntot], FLOAT), self.out([ntot], FLOAT)
            wi = (abi.sg_tensor * len(ws))(*[w.c() for w in ws])
            wc = wcat.c()
            bi = (abi.sg_tensor * len(bs))(*[b.with_shape(Shape([b.size()], [1], b.shape.offset)).c() for b in bs])
            bc = bcat.c()
            # the two concatenations, kept as replayable calls: they run again whenever parameters have
            # been rewritten since (an optimizer step), for this evaluation and for any recorded Program
            calls = [(self.lib.sg_concat, (1, wi, len(ws), C.byref(wc)), [wi, wc]), (self.lib.sg_concat, (0, bi, len(bs), C.byref(bc)), [bi, bc])]
            cache[key] = {"w": wcat, "b": bcat, "src": (ws, bs), "calls": calls, "epoch": None}  # sources kept: pointers stay unique
        entry = cache[key]
        refresh_derived(self.ctx, [entry])
        if self.record is not None and entry not in self.derived:
            self.derived.append(entry)
        wcat, bcat = entry["w"], entry["b"]
        a = self.get(a_node)
        if not a.is_dense():
            a = self.run_copy(a)
        M, ntot = a.extents[0], wcat.extents[1]
        y = self.out([M, ntot], FLOAT)
        epi = {"alpha": 1.0, "bias": bcat}
        keep = self.keepalive
        e = self._epi_struct(epi, keep)
        keep.append(e)
        ac, wc, yc = a.c(), wcat.c(), y.c()
        self.call(self.lib.sg_gemm, 0, 0, C.byref(ac), C.byref(wc), C.byref(yc), C.byref(e))
        off, mine = 0, None
        for top, g2, w2, _ in members:
            n = w2.value.extents[1]
            blk = y.with_shape(Shape([M, n], [ntot, 1], y.shape.offset + off))
            sh = blk.shape.reshape_view(top.extents)
            t = blk.with_shape(sh) if sh is not None else self.run_copy(blk).with_shape(Shape(top.extents))
            off += n
            if top is v:
                mine = t
            else:
                self.memo[id(top)] = t
                self.keep[id(top)] = top
        return mine

    def _match_res(self, v, chain):
        """(act?(core)) + R  in either order."""
        if v.op != "binary" or v.attrs["name"] != "add":
            return None, None
        l, r = v.inputs
        for y, res in ((l, r), (r, l)):
            if res.op == "expand" or res.extents != v.extents:
                continue
            sub = []
            act, x = self._match_act(y, sub)
            m = self._match_core(x, sub)
            if m is None or m["g"].size() != v.size():
                continue
            # the residual must not itself hang off the same GEMM
            if any(res is n for n in sub):
                continue
            if act is not None:
                m["act"] = act
                sub.append(y)
            chain.extend(sub)
            return m, res
        return None, None

    def try_permuted_matmul(self, v):
        """copy(permute(G)) with the last axis kept in place: let G write the permuted layout."""
        p = v.inputs[0]
        if p.op != "permute" or self.done(p) or self.n_users(p) != 1 or id(p) in self.targets:
            return None
        g = p.inputs[0]
        if g.op != "matmul_nd" or self.done(g) or self.n_users(g) != 1 or id(g) in self.targets:
            return None
        axes = p.attrs["axes"]
        if axes[-1] != g.rank - 1:
            return None
        y = self.out(v.extents, FLOAT)
        inv = [0] * len(axes)
        for i, a in enumerate(axes):
            inv[a] = i
        dest = y.with_shape(y.shape.permute(inv))  # g's extents over y's memory
        if self.try_attention(g, dest) is None:
            self.run_gemm(g, None, dest)
        return y

    # ---- fused row operators
    def _ev_softmax(self, v):
        x = v.inputs[0]
        addend = None
        if (_FUSION["on"] and x.op == "binary" and x.attrs["name"] == "add" and not self.done(x)
                and self.n_users(x) == 1 and id(x) not in self.targets):
            a, b = self.get(x.inputs[0]), self.get(x.inputs[1])
            if a.strides[-1] == 1 or a.extents[-1] == 1:
                xt, addend = a, b
            elif b.strides[-1] == 1:
                xt, addend = b, a
            else:
                xt = None
            if xt is None:
                xt = self.get(x)
                addend = None
        else:
            xt = self.get(x)
        if xt.strides[-1] != 1 and xt.extents[-1] != 1:
            xt = self.run_copy(xt)
        y = self.out(v.extents, FLOAT)
        xc, yc = xt.c(), y.c()
        ac = addend.c() if addend is not None else None
        self.call(self.lib.sg_softmax_lastaxis, C.byref(xc), C.byref(ac) if ac is not None else None, C.byref(yc))
        return y

    def _ev_softmax_ce(self, v):
        x, lab = self.get(v.inputs[0]), self.get(v.inputs[1])
        y = self.out(v.extents, FLOAT)
        xc, lc, yc = x.c(), lab.c(), y.c()
        self.call(self.lib.sg_softmax_cross_entropy, C.byref(xc), C.byref(lc), C.byref(yc))
        return y

    def _ev_layer_norm(self, v):
        x, g, b = (self.get(i) for i in v.inputs)
        if x.strides[-1] != 1 and x.extents[-1] != 1:
            x = self.run_copy(x)
        y = self.out(v.extents, FLOAT)
        xc, gc, bc, yc = x.c(), g.c(), b.c(), y.c()
        self.call(self.lib.sg_layer_norm_lastaxis, C.byref(xc), C.byref(gc), C.byref(bc), C.c_float(v.attrs["eps"]), C.byref(yc))
        return y
