"""Neural-network compositions: host-side mirror of ops/nn.rs and ops/metric.rs.

With fusion on (the default) softmax, softmax_cross_entropy and layer_norm over the LAST axis become
single graph nodes that the backend runs as one fused row kernel; in every other case — and always
with `var.set_fusion(False)` — they are the reference's compositions of maps and reductions, op for
op.  Both forms are compared against each other and against the CPU oracle by the parity tests.
"""
from . import abi
from .shape import Shape, norm_axes
from .tensor import FLOAT, UINT, INT
from .var import Var, fusion_enabled, gt, into_var


def relu(x):
    """nn.rs:33-40: float(x > 0) * x."""
    x = into_var(x)
    return gt(x, 0.0).float() * x


def gelu(x):
    """erf-GELU 0.5*x*(1+erf(x/sqrt 2)) from the reference's own maps (UnaryMap::Erf, map.rs:104)."""
    x = into_var(x)
    return (x * 0.5) * ((x / 1.4142135381698608).erf() + 1.0)


def softmax_composed(x, axes):
    """nn.rs:42-56."""
    x = into_var(x)
    axes = norm_axes(axes, x.rank)
    xm = x.max(axes, True)
    y = (x - xm).exp()
    s = y.sum(axes, True)
    return y / s


def softmax(x, axes):
    x = into_var(x)
    axes = norm_axes(axes, x.rank)
    if fusion_enabled() and axes == [x.rank - 1] and x.dtype == FLOAT:
        return Var(Shape(x.extents), FLOAT, "softmax", [x])
    return softmax_composed(x, axes)


def log_sum_exp(x, axes):
    """nn.rs:58-68."""
    x = into_var(x)
    axes = norm_axes(axes, x.rank)
    c = x.max(axes, True)
    return (x - c).exp().sum(axes, True).log() + c


def softmax_cross_entropy_composed(x1, x2):
    """nn.rs:70-82."""
    x1, x2 = into_var(x1), into_var(x2)
    log_z = x1 - log_sum_exp(x1, 1)
    log_p = log_z.gather(x2, 1)
    return -log_p.sum(1, False)


def softmax_cross_entropy(x1, x2):
    x1, x2 = into_var(x1), into_var(x2)
    if (fusion_enabled() and x1.rank == 2 and x2.rank == 2 and x2.extents == [x1.extents[0], 1]
            and x1.dtype == FLOAT and x2.dtype in (UINT, INT)):
        return Var(Shape([x1.extents[0]]), FLOAT, "softmax_ce", [x1, x2])
    return softmax_cross_entropy_composed(x1, x2)


def layer_norm_composed(x, axes, gamma, beta, eps):
    """nn.rs:84-100."""
    x = into_var(x)
    axes = norm_axes(axes, x.rank)
    m = x.mean(axes, True)
    v = x.var(axes, True)
    xc = (x - m) / (v + float(eps)).sqrt()
    return xc * gamma + beta


def layer_norm(x, axes, gamma, beta, eps):
    x, gamma, beta = into_var(x), into_var(gamma), into_var(beta)
    axes = norm_axes(axes, x.rank)
    n = x.extents[-1]
    ok = lambda p: p.size() == 1 or (p.size() == n and p.extents[-1] == n)
    if fusion_enabled() and axes == [x.rank - 1] and x.dtype == FLOAT and ok(gamma) and ok(beta):
        return Var(Shape(x.extents), FLOAT, "layer_norm", [x, gamma, beta], {"eps": float(eps)})
    return layer_norm_composed(x, axes, gamma, beta, eps)


def accuracy(logits, labels):
    """metric.rs:4-16: float(sum_0(argmax_1(logits, keep) == labels)) / B."""
    logits, labels = into_var(logits), into_var(labels)
    hit = logits.argmax(1, True)
    from .var import eq
    return eq(hit, labels).sum(0, False).float() / float(logits.extents[0])
