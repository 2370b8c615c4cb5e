"""Reverse-mode differentiation of a `Var` graph: host-side mirror of var.rs:44-103 and of the `grad`
method of every operator in ops/*.rs.

Like the reference, differentiation only BUILDS graphs: the gradient of each operator is written in
terms of the forward operators (map, reduce, gemm, gather/scatter, slice/unslice, im2col/col2im), so
the backward pass runs on the same kernels as the forward pass.  The rules below restate the
reference's, including the ones that are only right for special cases:

* `Permute::grad` applies the SAME permutation to gy (core.rs:388-393), which is the inverse only
  for involutions (every transpose is one);
* `TernaryMapOperator::grad` hands `cond(c, gy, 0)` to the condition, `cond(c, 0, gy)` to the first
  branch and nothing to the second (map.rs:1094-1099);
* `ReduceOperator::grad` for max/min routes gy to every element equal to the extremum
  (reduce.rs:250-251).

The fused nodes this package adds (softmax, softmax_ce, layer_norm, matmul_nd) have no counterpart
in the reference; they differentiate through the reference's own composition of the same function
(nn.rs:42-100, gemm.rs:53-104), so the gradient graph is the one the reference would build.
"""
import heapq
import math

from . import nn
from . import var as V
from .tensor import FLOAT
from .var import Var, scalar


def t_order(v, memo=None):
    """Operation::t_order (ops.rs:262-310): 0 for data and nullary operators, else 1 + max over inputs."""
    memo = {} if memo is None else memo
    stack = [v]
    while stack:
        n = stack[-1]
        if id(n) in memo:
            stack.pop()
            continue
        if not n.inputs:
            memo[id(n)] = 0
            stack.pop()
            continue
        todo = [i for i in n.inputs if id(i) not in memo]
        if todo:
            stack.extend(todo)
            continue
        memo[id(n)] = 1 + max(memo[id(i)] for i in n.inputs)
        stack.pop()
    return memo[id(v)]


def _zeros_like(x):
    return scalar(0.0, x.extents)


def _unary(name, x, y, gy):
    """UnaryMapOperator::grad (map.rs:937-968)."""
    if name in ("copy", "cast_int", "cast_float"):
        return gy
    if name == "abs":
        return V.sign(x) * gy
    if name == "neg":
        return -gy
    if name == "recip":
        return -gy / x.square()
    if name == "log":
        return gy / x
    if name == "exp":
        return gy * y
    if name == "sqrt":
        return gy / (y * 2.0)
    if name == "square":
        return gy * x * 2.0
    if name == "erf":
        return gy * float(2.0 / math.sqrt(math.pi)) / x.square().exp()
    if name in ("sign", "ceil", "floor", "round"):
        return _zeros_like(x)
    if name == "sin":
        return gy * x.cos()
    if name == "sinh":
        return gy * x.cosh()
    if name == "cos":
        return -gy * x.sin()
    if name == "cosh":
        return gy * x.sinh()
    if name == "tan":
        return gy / x.cos().square()
    if name == "tanh":
        return gy / x.cosh().square()
    if name == "asin":
        return gy / (-x.square() + 1.0).sqrt()
    if name == "asinh":
        return gy / (x.square() + 1.0).sqrt()
    if name == "acos":
        return -gy / (-x.square() + 1.0).sqrt()
    if name == "acosh":
        return gy / (x.square() - 1.0).sqrt()
    if name == "atan":
        return gy / (x.square() + 1.0)
    if name == "atanh":
        return gy / (-x.square() + 1.0)
    if name == "not":
        return None
    raise ValueError(f"no gradient rule for unary map {name}")


def _binary(name, x0, x1, gy):
    """BinaryMapOperator::grad (map.rs:1014-1041)."""
    if name == "add":
        return [gy, gy]
    if name == "sub":
        return [gy, -gy]
    if name == "div":
        return [gy / x1, gy * (-x0 / x1.square())]
    if name == "mul":
        return [gy * x1, gy * x0]
    if name == "mod":
        return [gy, -gy * (x0 / x1).floor()]
    if name == "pow":
        return [gy * x1 * x0.pow(x1 - 1.0), gy * x0.pow(x1) * x0.log()]
    if name == "min":
        return [gy * V.lt(x0, x1).float(), gy * V.ge(x0, x1).float()]
    if name == "max":
        return [gy * V.lt(x1, x0).float(), gy * V.ge(x1, x0).float()]
    return [None, None]  # and, or, eq, ne, gt, ge, lt, le


def _gemm(x, gy, ta, tb, mm):
    """Gemm::grad / GemmBatched::grad (gemm.rs:151-160, 301-320)."""
    if not ta and not tb:
        return [mm(gy, x[1], False, True), mm(x[0], gy, True, False)]
    if not ta and tb:
        return [mm(gy, x[1], False, False), mm(gy, x[0], True, False)]
    if ta and not tb:
        return [mm(x[1], gy, False, True), mm(x[0], gy, False, False)]
    return [mm(x[1], gy, True, True), mm(gy, x[0], True, True)]


def _through_composition(v, gy, composed):
    """Gradient of a fused node = gradient of the reference's composition on the same inputs."""
    ins = list(v.inputs)
    g = grad(composed, ins, seed=gy, allow_unreached=True)
    return g


def op_grad(v, gy):
    """Operation::grad (ops.rs:326-336): one entry (a Var or None) per input of `v`."""
    op, x, a = v.op, v.inputs, v.attrs
    if op in ("literal", "data", "rand_uniform", "rand_normal"):  # nullary (rand.rs:59, 102)
        return []
    if op == "unary":
        return [_unary(a["name"], x[0], v, gy)]
    if op == "binary":
        return _binary(a["name"], x[0], x[1], gy)
    if op == "cond":
        return [V.cond(x[0], gy, 0.0), V.cond(x[0], 0.0, gy), None]
    if op == "reshape":  # core.rs:245-247
        return [V.reshape(gy, x[0].shape)]
    if op == "expand":   # core.rs:292-313
        surplus = gy.rank - x[0].rank
        axes = list(range(surplus)) + [i + surplus for i in range(x[0].rank) if gy.extents[i + surplus] != x[0].extents[i]]
        if not axes:
            return [gy.view(x[0].extents)]
        return [gy.sum(axes, False).view(x[0].extents)]
    if op == "permute":  # core.rs:388-393
        return [V.permute(gy, a["axes"])]
    if op == "squeeze":  # core.rs:430-432
        return [V.unsqueeze(gy, a["axis"])]
    if op == "unsqueeze":  # core.rs:469-471
        return [V.squeeze(gy, a["axis"])]
    if op == "slice":    # core.rs:510-518
        return [V.unslice(gy, a["axis"], a["start"], x[0].extents[a["axis"]])]
    if op == "unslice":  # core.rs:562-569
        return [V.slice_(gy, a["axis"], a["start"], a["start"] + x[0].extents[a["axis"]])]
    if op == "gather":   # core.rs:651-653
        return [V.scatter(gy, x[1], a["axis"], x[0].extents), None]
    if op == "scatter":  # core.rs:760-762
        return [V.gather(gy, x[1], a["axis"]), None]
    if op == "concat":   # core.rs:882-890
        out, i = [], 0
        for xi in x:
            e = xi.extents[a["axis"]]
            out.append(V.slice_(gy, a["axis"], i, i + e))
            i += e
        return out
    if op == "reduce":   # reduce.rs:236-253
        x0 = x[0]
        ext = V.reduced_extents(x0.extents, a["axes"], True)
        y, g = v, gy
        if v.extents != ext:
            y, g = v.view(ext), gy.view(ext)
        kind = a["op"]
        if kind == "sum":
            return [g.expand(x0.extents)]
        if kind == "prod":
            return [g * y / x0]
        return [V.cond(V.eq(x0, y), g, 0.0)]
    if op == "reduce_arg":  # reduce.rs:365-367
        return [None]
    if op == "gemm":
        return _gemm(x, gy, a["ta"], a["tb"], V.gemm)
    if op == "gemm_batched":
        return _gemm(x, gy, a["ta"], a["tb"], V.gemm_batched)
    if op == "im2col":   # conv.rs:275-287
        return [V.col2im(gy, [x[0].extents[2], x[0].extents[1]], a["ker"], a["stride"], a["pad"], a["dil"])]
    if op == "col2im":   # conv.rs:386-394
        return [V.im2col(gy, a["ker"], a["stride"], a["pad"], a["dil"])]
    # ---- fused nodes of this package: differentiate the reference's composition
    if op == "softmax":
        return _through_composition(v, gy, nn.softmax_composed(x[0], [x[0].rank - 1]))
    if op == "softmax_ce":
        return _through_composition(v, gy, nn.softmax_cross_entropy_composed(x[0], x[1]))
    if op == "layer_norm":
        return _through_composition(v, gy, nn.layer_norm_composed(x[0], [x[0].rank - 1], x[1], x[2], a["eps"]))
    if op == "matmul_nd":
        return _through_composition(v, gy, V.matmul_batched_composed(x[0], x[1]))
    raise ValueError(f"no gradient rule for operator {op}")


def grad(y, xs, seed=None, allow_unreached=False):
    """var.rs:56-103.  Returns the gradients of `y` with respect to each Var of `xs`, in order.
    The walk pops the deepest pending node first, so a node's gradient is complete (summed over all
    its consumers) before it is propagated.  `seed` replaces the all-ones gy/gy.  A variable `y` does
    not depend on makes the reference panic (unwrap of a missing entry, var.rs:99); here that is a
    KeyError unless `allow_unreached`, which yields None for it."""
    xs = list(xs)
    memo = {}
    grads = {id(y): seed if seed is not None else scalar(1.0, y.extents)}
    nodes = {id(y): y}
    heap, counter = [(-t_order(y, memo), 0, id(y))], 1
    while heap:
        _, _, key = heapq.heappop(heap)
        node = nodes[key]
        if not node.inputs or node.op == "data":
            continue
        gy = grads[key]
        for xi, gx in zip(node.inputs, op_grad(node, gy)):
            if gx is None:
                continue
            if gx.extents != xi.extents:
                raise AssertionError(f"grad shape error at {node.op}: {gx.extents} for an input of {xi.extents}")
            if id(xi) not in grads:
                nodes[id(xi)] = xi
                heapq.heappush(heap, (-t_order(xi, memo), counter, id(xi)))
                counter += 1
                grads[id(xi)] = gx
            else:
                grads[id(xi)] = gx + grads[id(xi)]
    out = []
    for x in xs:
        if id(x) not in grads:
            if allow_unreached:
                out.append(None)
                continue
            raise KeyError("grad: y does not depend on one of the requested variables")
        out.append(grads[id(x)])
    return out


def grad_param(y, model):
    """var.rs:46-54: gradients with respect to every parameter of a layer, as {param: grad} in
    parameter order (the reference's HashMap has no order; Python dicts keep this one)."""
    params = model.params()
    return dict(zip(params, grad(y, params)))


def grad_check(y, x, err, ctx, eps=1e-4):
    """var.rs:107-160: compare x.grad(y) with central finite differences of sum(y), element by element.
    Returns True when every |analytic - numeric| < err."""
    import numpy as np
    from .tensor import Tensor
    gx = grad(y, [x])[0].eval(ctx).numpy()
    base = x.value.numpy().astype(np.float32)
    flat = base.reshape(-1).copy()
    num = np.zeros_like(flat, dtype=np.float64)

    def total(arr):
        x.set(Tensor.from_numpy(ctx, arr.reshape(base.shape)))
        return float(V.evaluate_fresh(ctx, [y])[0].numpy().astype(np.float64).sum())

    for i in range(flat.size):
        keep = flat[i]
        flat[i] = keep + eps
        hi = total(flat)
        flat[i] = keep - eps
        lo = total(flat)
        flat[i] = keep
        num[i] = (hi - lo) / (2 * eps)
    x.set(Tensor.from_numpy(ctx, base))
    return bool(np.max(np.abs(gx.reshape(-1).astype(np.float64) - num)) < err)
