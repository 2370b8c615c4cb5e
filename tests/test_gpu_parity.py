"""Parity of the HIP path (through the C ABI) with the CPU oracle on seeded random inputs.

Bar: indexing, gather, argmax, compare/logic results and pure +,-,*,/ arithmetic are bit-exact;
transcendental maps and reductions agree within rel 1e-4; GEMM, convolution and model outputs
within rel 1e-3 (tests/util.py).  Every test prints its case before touching the GPU.
"""
import ctypes as C

import numpy as np
import pytest

import sage_amd as S
from oracle import oracle as O
from sage_amd import abi, nn
from sage_amd import var as V
from tests.util import REL_GEMM, REL_MAP, close, exact

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = S.Context()
    yield c
    c.close()


@pytest.fixture
def ctx_under(monkeypatch):
    """ctx_under(NAME=value, ..) -> a context created AFTER those environment switches were set: the library reads its
    measurement switches once, when a context is created."""
    made = []

    def make(**env):
        for k, v in env.items():
            monkeypatch.setenv(k, v)
        made.append(S.Context())
        return made[-1]
    yield make
    for c in made:
        c.close()


@pytest.fixture(autouse=True)
def _fusion_on():
    V.set_fusion(True)
    yield
    V.set_fusion(True)


def say(*a):
    print("[case]", *a, flush=True)


def dev(ctx, a):
    return S.Var.new(S.Tensor.from_numpy(ctx, a))


def ht(a):
    return O.HT.from_numpy(a)


def view_pair(ctx, a, fn):
    """The same layout operation applied to a device Var and to an oracle host tensor."""
    return fn(dev(ctx, a)), fn(ht(a))


# ----------------------------------------------------------------------------- maps
UNARY_DOMAIN = {
    "log": (0.1, 4.0), "sqrt": (0.0, 4.0), "acosh": (1.0, 5.0), "atanh": (-0.95, 0.95),
    "asin": (-1.0, 1.0), "acos": (-1.0, 1.0), "recip": (0.5, 3.0), "exp": (-5.0, 5.0),
}
EXACT_UNARY = {"copy", "abs", "neg", "recip", "sqrt", "square", "sign", "ceil", "floor", "round", "cast_int", "cast_float", "not"}


@pytest.mark.parametrize("name", abi.UNARY)
@pytest.mark.parametrize("shape", [(64, 256), (7, 13), (3, 5, 4)], ids=["vec", "odd", "rank3"])
def test_unary_maps(ctx, name, shape):
    say("unary", name, shape)
    rng = np.random.default_rng(100 + abi.UNARY.index(name))
    lo, hi = UNARY_DOMAIN.get(name, (-3.0, 3.0))
    x = rng.uniform(lo, hi, shape).astype(np.float32)
    if name in ("sign", "ceil", "floor", "round", "abs"):
        x.flat[:6] = [0.0, -0.0, 0.5, -0.5, 1.5, -2.5]
    y = V.unary_map(dev(ctx, x), name).eval(ctx).numpy()
    y_or = O.unary(name, ht(x)).numpy()
    assert y.dtype == y_or.dtype
    if name in EXACT_UNARY:
        exact(y, y_or, name)
    else:
        close(y, y_or, REL_MAP, name)


@pytest.mark.parametrize("name", [b for b in abi.BINARY if b != "mod"])
def test_binary_maps_float(ctx, name):
    say("binary float", name)
    rng = np.random.default_rng(7)
    a = rng.uniform(0.2, 3.0, (33, 20)).astype(np.float32)
    b = rng.uniform(0.2, 3.0, (33, 20)).astype(np.float32)
    b[::3] = a[::3]  # ties for the comparisons
    y = V.binary_map(dev(ctx, a), dev(ctx, b), name).eval(ctx).numpy()
    y_or = O.binary(name, ht(a), ht(b)).numpy()
    assert y.dtype == y_or.dtype
    if name == "pow":
        close(y, y_or, REL_MAP, name)
    else:
        exact(y, y_or, name)


@pytest.mark.parametrize("name", ["add", "sub", "mul", "div", "min", "max", "eq", "lt", "ge", "and", "or"])
@pytest.mark.parametrize("dt", [np.int32, np.uint32])
def test_binary_maps_int(ctx, name, dt):
    say("binary int", name, dt.__name__)
    rng = np.random.default_rng(11)
    a = rng.integers(0 if dt == np.uint32 else -50, 50, (16, 12)).astype(dt)
    b = rng.integers(1, 9, (16, 12)).astype(dt)
    y = V.binary_map(dev(ctx, a), dev(ctx, b), name).eval(ctx).numpy()
    exact(y, O.binary(name, ht(a), ht(b)).numpy(), name)


def test_int_unary_and_casts(ctx):
    say("int unary / casts")
    a = np.array([[-7, 0, 3, 2147483647], [5, -1, 9, -2147483648]], dtype=np.int32)
    for name in ("neg", "copy", "not", "cast_float", "cast_int"):
        exact(V.unary_map(dev(ctx, a), name).eval(ctx).numpy(), O.unary(name, ht(a)).numpy(), name)
    f = np.array([[-2.7, -0.2, 0.0, 0.9], [1.5, 2.5, 100.25, -100.75]], dtype=np.float32)
    exact(V.unary_map(dev(ctx, f), "cast_int").eval(ctx).numpy(), np.trunc(f).astype(np.int32), "trunc toward zero")
    u = np.array([[0, 1, 2, 4000000000]], dtype=np.uint32)
    exact(V.unary_map(dev(ctx, u), "cast_float").eval(ctx).numpy(), O.unary("cast_float", ht(u)).numpy(), "uint->float")


LAYOUTS = {
    "transpose01": lambda t: t.transpose(0, 1),
    "permute_201": lambda t: t.permute([2, 0, 1]),
    "slice_mid": lambda t: t.slice(1, 1, 4),
    "slice_last": lambda t: t.slice(2, 3, 11),
    "row_broadcast": lambda t: t.slice(2, 0, 1).expand(list(t.extents)),
    "col_broadcast": lambda t: t.slice(1, 0, 1).expand(list(t.extents)),
    "index_expand": lambda t: t.index(0, 1).expand(list(t.extents)),
}


@pytest.mark.parametrize("layout", list(LAYOUTS))
def test_map_operand_layouts(ctx, layout):
    """Every index-translation class: direct, permuted, offset windows, stride-0 broadcasts."""
    say("layout", layout)
    rng = np.random.default_rng(3)
    a = rng.standard_normal((6, 8, 12)).astype(np.float32)
    xd, xo = view_pair(ctx, a, LAYOUTS[layout])
    b = rng.standard_normal(tuple(xo.extents)).astype(np.float32)
    exact(xd.copy().eval(ctx).numpy(), xo.numpy(), "copy")
    yd = (xd * dev(ctx, b) + xd).eval(ctx).numpy()
    yo = O.binary("add", O.binary("mul", xo, ht(b)), xo).numpy()
    exact(yd, yo, "x*b+x")


def test_map_vector_and_broadcast_paths(ctx):
    """Shapes that take the 16-byte path: bias rows, per-row scalars, attention-mask broadcast."""
    rng = np.random.default_rng(5)
    x = rng.standard_normal((96, 128)).astype(np.float32)
    bias = rng.standard_normal((128,)).astype(np.float32)
    rowv = rng.standard_normal((96, 1)).astype(np.float32)
    say("bias add")
    exact((dev(ctx, x) + dev(ctx, bias)).eval(ctx).numpy(), x + bias, "x+bias")
    say("exp(x - rowmax)")
    y = (dev(ctx, x) - dev(ctx, rowv)).exp().eval(ctx).numpy()
    close(y, O.unary("exp", O.binary("sub", ht(x), ht(rowv))).numpy(), REL_MAP, "exp(x-c)")
    say("scores/8 + mask")
    s = rng.standard_normal((4, 3, 16, 16)).astype(np.float32)
    m = rng.integers(0, 2, (4, 16)).astype(np.float32)
    md = (-dev(ctx, m).view([4, 1, 1, 16]) + 1.0) * -1e5
    mo = O.binary("mul", O.binary("add", O.unary("neg", ht(m).view([4, 1, 1, 16])), 1.0), -1e5)
    exact((dev(ctx, s) / 8.0 + md).eval(ctx).numpy(), O.binary("add", O.binary("div", ht(s), 8.0), mo).numpy(), "s/8+mask")
    say("five-input layer-norm tail")
    mean = rng.standard_normal((96, 1)).astype(np.float32)
    den = rng.uniform(0.5, 2.0, (96, 1)).astype(np.float32)
    g, b = np.float32(1.5), np.float32(-0.25)
    yd = ((dev(ctx, x) - dev(ctx, mean)) / dev(ctx, den) * dev(ctx, np.array([g])) + dev(ctx, np.array([b]))).eval(ctx).numpy()
    exact(yd, ((x - mean) / den * g + b).astype(np.float32), "ln tail")


def test_map_errors(ctx):
    say("map error behaviour")
    a = dev(ctx, np.ones((2, 3), np.float32))
    i = dev(ctx, np.ones((2, 3), np.int32))
    with pytest.raises(abi.DTypeError):
        V.binary_map(a, i, "add")          # map.rs:489
    with pytest.raises(abi.DTypeError):
        V.cond(a, a, a)                    # map.rs:870: condition must be uint
    with pytest.raises(abi.SageError):
        V.binary_map(a, a, "mod").eval(ctx)  # map.rs:275: mod() cannot be built
    with pytest.raises(ValueError):
        V.binary_map(a, dev(ctx, np.ones((2, 4), np.float32)), "add")  # shape::union InvalidBroadcast


def test_fused_map_equals_unfused(ctx):
    say("fused vs unfused map chain")
    rng = np.random.default_rng(9)
    x = rng.standard_normal((40, 64)).astype(np.float32)
    y = rng.uniform(0.5, 2.0, (40, 64)).astype(np.float32)

    def build():
        a, b = dev(ctx, x), dev(ctx, y)
        return V.cond(V.gt(a, 0.0), (a * b + 1.0).sqrt() / b, -a.abs() * 0.5)

    n0 = ctx.launches
    f = build().eval(ctx).numpy()
    assert ctx.launches - n0 == 1
    V.set_fusion(False)
    u = build().eval(ctx).numpy()
    exact(f, u, "fusion changes no value")


# ----------------------------------------------------------------------------- reductions
RED_CASES = [
    ((8, 1024), [1]), ((8, 1024), [0]), ((5, 37), [1]), ((3, 5000), [1]), ((64, 9, 32), [1]),
    ((2, 3, 2, 3, 2), [0, 2, 3]), ((6, 7, 8), [0, 1, 2]), ((4, 6, 10), [2, 0]), ((128, 128), [1]), ((1, 7), [0]),
    # few contiguous outputs, long strided reduced axis (bias gradients): chunked column path
    ((5000, 70), [0]), ((6272, 64), [0]), ((3, 400, 513), [0, 1]), ((300, 16), [0]),
    # row lengths that leave some lanes out of the four-loads-per-trip loop and in its one-load tail
    ((7, 1000), [1]), ((4, 1900), [1]), ((3, 2052), [1]),
]


@pytest.mark.parametrize("op", ["sum", "prod", "max", "min"])
@pytest.mark.parametrize("init", ["ref_zero", "identity"])
@pytest.mark.parametrize("case", range(len(RED_CASES)))
def test_reduce(ctx, op, init, case):
    shape, axes = RED_CASES[case]
    say("reduce", op, init, shape, axes)
    rng = np.random.default_rng(case)
    x = rng.uniform(0.7, 1.3, shape).astype(np.float32) * rng.choice([-1.0, 1.0], shape).astype(np.float32)
    if op == "prod":
        x = np.abs(x)
    for keep in (False, True):
        y = V.reduce(dev(ctx, x), axes, keep, op, init).eval(ctx).numpy()
        y_or = O.reduce(ht(x), axes, keep, op, O.INIT_REF_ZERO if init == "ref_zero" else O.INIT_IDENTITY).numpy()
        if op in ("max", "min"):
            exact(y, y_or, f"{op} keep={keep}")
        else:
            close(y, y_or, REL_MAP, f"{op} keep={keep}")


def test_reduce_reference_zero_accumulator(ctx):
    """reduce.rs:282: max of an all-negative row is 0, min of an all-positive row is 0, prod is 0."""
    say("reduce ref_zero semantics")
    x = np.array([[-3.0, -1.0, -2.0], [4.0, 2.0, 9.0]], dtype=np.float32)
    exact(V.max_(dev(ctx, x), 1).eval(ctx).numpy(), np.array([0.0, 9.0], np.float32), "max")
    exact(V.min_(dev(ctx, x), 1).eval(ctx).numpy(), np.array([-3.0, 0.0], np.float32), "min")
    exact(V.prod(dev(ctx, x), 1).eval(ctx).numpy(), np.array([-0.0, 0.0], np.float32), "prod")
    exact(V.reduce(dev(ctx, x), 1, False, "max", "identity").eval(ctx).numpy(), np.array([-1.0, 9.0], np.float32), "true max")


def test_reduce_strided_and_int(ctx):
    rng = np.random.default_rng(21)
    a = rng.standard_normal((12, 10, 8)).astype(np.float32)
    for name in ("transpose01", "slice_mid", "permute_201"):
        say("reduce over", name)
        xd, xo = view_pair(ctx, a, LAYOUTS[name])
        for axes in ([0], [1], [2], [0, 2]):
            close(xd.sum(axes).eval(ctx).numpy(), O.rsum(xo, axes).numpy(), REL_MAP, f"{name} {axes}")
    say("reduce int")
    i = rng.integers(-20, 20, (9, 33)).astype(np.int32)
    exact(dev(ctx, i).sum(1).eval(ctx).numpy(), O.rsum(ht(i), 1).numpy(), "int sum")
    exact(dev(ctx, i).max(0).eval(ctx).numpy(), O.rmax(ht(i), 0).numpy(), "int max")
    j = rng.integers(-20, 20, (4000, 40)).astype(np.int32)
    exact(dev(ctx, j).sum(0).eval(ctx).numpy(), O.rsum(ht(j), 0).numpy(), "int column sum")
    exact(dev(ctx, j).min(0).eval(ctx).numpy(), O.rmin(ht(j), 0).numpy(), "int column min")


@pytest.mark.parametrize("shape,axis", [((2, 3, 4), 1), ((64, 1000), 1), ((64, 1000), 0), ((5, 7, 300), 2), ((9, 64), 1), ((3, 1), 1)])
@pytest.mark.parametrize("op", ["max", "min"])
def test_reduce_arg(ctx, shape, axis, op):
    say("reduce_arg", op, shape, axis)
    rng = np.random.default_rng(4)
    x = rng.integers(-6, 6, shape).astype(np.float32)  # many ties: first index must win
    for keep in (False, True):
        y = V.reduce_arg(dev(ctx, x), axis, keep, op).eval(ctx).numpy()
        exact(y, O.reduce_arg(ht(x), axis, keep, op).numpy(), f"arg{op}")
    xt_d, xt_o = view_pair(ctx, x, lambda t: t.transpose(0, 1))
    ax = {0: 1, 1: 0}.get(axis, axis)
    exact(V.reduce_arg(xt_d, ax, False, op).eval(ctx).numpy(), O.reduce_arg(xt_o, ax, False, op).numpy(), "transposed")


def test_mean_var_accuracy(ctx):
    say("mean / var / accuracy")
    rng = np.random.default_rng(8)
    x = rng.standard_normal((6, 50)).astype(np.float32)
    close(dev(ctx, x).mean(1, True).eval(ctx).numpy(), O.mean(ht(x), 1, True).numpy(), REL_MAP, "mean")
    close(dev(ctx, x).var(1, True).eval(ctx).numpy(), O.var(ht(x), 1, True).numpy(), 1e-3, "var")
    logits = rng.standard_normal((64, 10)).astype(np.float32)
    labels = rng.integers(0, 10, (64, 1)).astype(np.uint32)
    acc = nn.accuracy(dev(ctx, logits), dev(ctx, labels)).eval(ctx).numpy()
    assert float(acc[0]) == float(np.mean(np.argmax(logits, 1) == labels[:, 0]))


# ----------------------------------------------------------------------------- indexing
def test_gather_scatter(ctx):
    rng = np.random.default_rng(12)
    x = rng.standard_normal((5, 6, 7)).astype(np.float32)
    for axis in range(3):
        say("gather axis", axis)
        shp = [3, 4, 5]
        ind = rng.integers(0, x.shape[axis], shp).astype(np.uint32)
        exact(V.gather(dev(ctx, x), dev(ctx, ind), axis).eval(ctx).numpy(), O.gather(ht(x), ht(ind), axis).numpy(), "gather")
    say("gather embedding (stride-0 index)")
    w = rng.standard_normal((50, 16)).astype(np.float32)
    ids = rng.integers(0, 50, (3, 9)).astype(np.int32)
    from sage_amd.layers import Embedding
    emb = Embedding(50, 16)
    emb.weight.set(S.Tensor.from_numpy(ctx, w))
    exact(emb.pass_(dev(ctx, ids)).eval(ctx).numpy(), w[ids], "embedding")
    exact(O.embedding(ht(w), ht(ids)).numpy(), w[ids], "oracle embedding")
    say("gather rows: 16-byte row path (wide table view, repeated ids) and its fallbacks (odd width, odd offset)")
    big = rng.standard_normal((40, 24)).astype(np.float32)
    ids2 = rng.integers(0, 40, (11,)).astype(np.uint32)
    ids2[3] = ids2[7]
    for lo, width in ((4, 16), (8, 12), (0, 24), (3, 16), (4, 10)):   # column window of the table: offset, width
        table = dev(ctx, big).slice(1, lo, lo + width)
        idx = dev(ctx, ids2).view([11, 1]).expand([11, width])
        exact(table.gather(idx, 0).eval(ctx).numpy(), big[ids2, lo:lo + width], f"gather rows lo={lo} width={width}")
    say("gather from a transposed table")
    xd, xo = view_pair(ctx, x, lambda t: t.transpose(0, 2))
    ind = rng.integers(0, 7, (7, 6, 2)).astype(np.uint32)
    exact(V.gather(xd, dev(ctx, ind), 0).eval(ctx).numpy(), O.gather(xo, ht(ind), 0).numpy(), "gather strided")
    say("scatter, unique indices")
    src = rng.standard_normal((4, 1)).astype(np.float32)
    ind = rng.integers(0, 10, (4, 1)).astype(np.uint32)
    exact(V.scatter(dev(ctx, src), dev(ctx, ind), 1, [4, 10]).eval(ctx).numpy(), O.scatter(ht(src), ht(ind), 1, [4, 10]).numpy(), "scatter")
    say("scatter, duplicate indices (atomic sum)")
    src = rng.standard_normal((64, 3)).astype(np.float32)
    ind = rng.integers(0, 4, (64, 3)).astype(np.uint32)
    want = np.zeros((4, 3), np.float64)
    for r in range(64):
        for c in range(3):
            want[ind[r, c], c] += src[r, c]
    close(V.scatter(dev(ctx, src), dev(ctx, ind), 0, [4, 3]).eval(ctx).numpy(), want, 1e-5, "scatter dup")


def test_unslice_concat(ctx):
    rng = np.random.default_rng(13)
    x = rng.standard_normal((4, 3, 5)).astype(np.float32)
    for axis, start, end in ((0, 2, 9), (1, 0, 3), (2, 1, 8)):
        say("unslice", axis, start, end)
        exact(V.unslice(dev(ctx, x), axis, start, end).eval(ctx).numpy(), O.unslice(ht(x), axis, start, end).numpy(), "unslice")
    say("concat incl. a strided input")
    a, b = rng.standard_normal((3, 2, 4)).astype(np.float32), rng.standard_normal((3, 5, 4)).astype(np.float32)
    c = rng.standard_normal((4, 3, 4)).astype(np.float32)
    cd, co = view_pair(ctx, c, lambda t: t.transpose(0, 1))
    exact(V.concat([dev(ctx, a), dev(ctx, b), cd], 1).eval(ctx).numpy(), O.concat([ht(a), ht(b), co], 1).numpy(), "concat")


def _random_view(rng, ext):
    """A host array and a layout operation (for view_pair) whose result has extents `ext`: the array is stored with its
    axes permuted, with room for a slice along one axis, and with some extent-1 axes broadcast to their extent."""
    rank = len(ext)
    perm = [int(p) for p in rng.permutation(rank)]          # stored axis i holds logical axis perm[i]
    stored = [ext[p] for p in perm]
    cut = int(rng.integers(0, rank))                            # stored axis that is sliced out of a larger one
    lo = int(rng.integers(0, 3))
    stored[cut] += lo + int(rng.integers(0, 3))
    bcast = [a for a in range(rank) if ext[a] > 1 and rng.uniform() < 0.2]   # logical axes stored with extent 1
    for a in bcast:
        if perm.index(a) != cut:
            stored[perm.index(a)] = 1
    inv = [perm.index(a) for a in range(rank)]

    def fn(t):
        t = t.slice(cut, lo, lo + (1 if stored[cut] == 1 else ext[perm[cut]]))
        t = t.permute(inv)
        return t.expand(list(ext))
    return stored, fn


def test_index_kernels_on_random_views(ctx):
    """gather, scatter, unslice and concat over 30 seeded random cases of rank 1..6: operands stored permuted, as windows of
    larger arrays and with broadcast axes, so that the host-side collapse of the index space meets merged, unmergeable and
    vanishing axes around the gather / scatter axis.  Integer data, so every result (duplicate scatter targets included)
    is exact against the oracle, whose index arithmetic is pinned by explicit loops on the CPU."""
    rng = np.random.default_rng(2024)
    for case in range(30):
        rank = int(rng.integers(1, 7))
        ext = [int(rng.integers(1, 6)) for _ in range(rank)]
        axis = int(rng.integers(0, rank))
        say("index kernels on random views", case, ext, axis)
        # gather: x's extents >= ind's except along the axis
        xext = [e + int(rng.integers(0, 3)) for e in ext]
        xext[axis] = int(rng.integers(1, 7))
        xs, xfn = _random_view(rng, xext)
        isz, ifn = _random_view(rng, ext)
        x = rng.integers(0, 1 << 20, xs).astype(np.uint32)
        ind = rng.integers(0, xext[axis], isz).astype(np.uint32)
        (xd, xo), (idd, ido) = view_pair(ctx, x, xfn), view_pair(ctx, ind, ifn)
        exact(V.gather(xd, idd, axis).eval(ctx).numpy(), O.gather(xo, ido, axis).numpy(), f"gather case {case}")
        # scatter: ind dense (the reference decomposes by ind's own strides), x any view with ind's extents, duplicates allowed
        oext = [e + int(rng.integers(0, 2)) for e in ext]
        oext[axis] = int(rng.integers(1, 5))
        ss, sfn = _random_view(rng, ext)
        src = rng.integers(0, 1000, ss).astype(np.uint32)
        ind2 = rng.integers(0, oext[axis], ext).astype(np.uint32)
        sd, so = view_pair(ctx, src, sfn)
        exact(V.scatter(sd, dev(ctx, ind2), axis, oext).eval(ctx).numpy(), O.scatter(so, ht(ind2), axis, oext).numpy(), f"scatter case {case}")
        # unslice and concat along the axis
        start = int(rng.integers(0, 3))
        end = start + ext[axis] + int(rng.integers(0, 3))
        exact(V.unslice(sd, axis, start, end).eval(ctx).numpy(), O.unslice(so, axis, start, end).numpy(), f"unslice case {case}")
        other = list(ext)
        other[axis] = int(rng.integers(1, 4))
        b = rng.integers(0, 1000, other).astype(np.uint32)
        exact(V.concat([sd, dev(ctx, b), sd], axis).eval(ctx).numpy(), O.concat([so, ht(b), so], axis).numpy(), f"concat case {case}")


# ----------------------------------------------------------------------------- GEMM
@pytest.mark.parametrize("mkn", [(1, 1, 1), (7, 13, 5), (128, 128, 128), (130, 257, 70), (64, 49, 64), (256, 64, 96), (33, 300, 200), (1, 512, 10), (300, 1, 17)])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_gemm_modes(ctx, mkn, ta, tb):
    m, k, n = mkn
    say("gemm", mkn, ta, tb)
    rng = np.random.default_rng(m * 7 + n)
    a = rng.uniform(-1, 1, (k, m) if ta else (m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (n, k) if tb else (k, n)).astype(np.float32)
    y = V.gemm(dev(ctx, a), dev(ctx, b), ta, tb).eval(ctx).numpy()
    close(y, O.gemm(ht(a), ht(b), ta, tb).numpy(), REL_GEMM, "gemm")
    ref64 = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
    close(y, ref64, REL_GEMM, "gemm vs float64")


@pytest.mark.parametrize("mkn,split", [((128, 4608, 512), None), ((512, 2304, 256), None), ((64, 1024, 64), None),
                                       ((70, 999, 33), "5"), ((130, 257, 70), "3"), ((128, 512, 128), "32"), ((37, 2000, 41), "7")])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, True)])
def test_gemm_split_k(ctx, ctx_under, mkn, split, ta, tb):
    """Few output tiles and a long K: the k range is split over workgroups and summed by a second kernel
    (chosen by itself for the first three shapes, forced for the ragged ones), with the epilogue behind it."""
    m, k, n = mkn
    say("gemm split-K", mkn, split, ta, tb)
    if split:
        ctx = ctx_under(SAGE_GEMM_SPLITK=split)
    rng = np.random.default_rng(m + k + n)
    a = rng.uniform(-1, 1, (k, m) if ta else (m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (n, k) if tb else (k, n)).astype(np.float32)
    bias = rng.uniform(-1, 1, (n,)).astype(np.float32)
    res = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    n0 = ctx.launches
    y = nn.relu(V.gemm(dev(ctx, a), dev(ctx, b), ta, tb) + dev(ctx, bias)).eval(ctx).numpy()
    assert ctx.launches - n0 == 1
    ref64 = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
    close(y, np.maximum(ref64 + bias, 0), REL_GEMM, "relu(gemm + bias) vs float64")
    close(y, O.relu(O.binary("add", O.gemm(ht(a), ht(b), ta, tb), ht(bias).expand([m, n]))).numpy(), REL_GEMM, "vs oracle")
    y2 = ((V.gemm(dev(ctx, a), dev(ctx, b), ta, tb) + dev(ctx, bias)) + dev(ctx, res)).eval(ctx).numpy()
    close(y2, ref64 + bias + res, REL_GEMM, "gemm + bias + residual vs float64")
    # the split is summed in a fixed order: the same call gives the same bits
    y3 = ((V.gemm(dev(ctx, a), dev(ctx, b), ta, tb) + dev(ctx, bias)) + dev(ctx, res)).eval(ctx).numpy()
    exact(y2, y3, "run-to-run")


@pytest.mark.parametrize("mkn", [(3200, 64, 3840), (3201, 96, 3838), (4096, 32, 2304)])
def test_gemm_more_tiles_than_resident_workgroups(ctx, mkn):
    """Outputs of 750..1000 tiles: more than the three workgroups per compute unit that fit at once, so
    workgroups take a second tile (exactly tiled shapes through buffer loads, the ragged one through the
    guarded loads).  Every element against float64, and the same bits on a second run."""
    m, k, n = mkn
    say("gemm tile walk", mkn)
    rng = np.random.default_rng(m + n)
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    bias = rng.uniform(-1, 1, (n,)).astype(np.float32)
    res = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    run = lambda: ((dev(ctx, a).matmul(dev(ctx, b)) + dev(ctx, bias)) + dev(ctx, res)).eval(ctx).numpy()
    y = run()
    close(y, a.astype(np.float64) @ b.astype(np.float64) + bias + res, REL_GEMM, "vs float64")
    exact(y, run(), "run-to-run")


def test_gemm_random_shapes_and_layouts(ctx):
    """Sixty seeded random products: extents 1..400 (most of them ragged against every tile size), all four
    transpose modes, operands that are row windows of larger matrices (element offsets, ld > width), with
    and without bias / ReLU / residual.  Against float64 and against the oracle."""
    rng = np.random.default_rng(2024)
    for case in range(60):
        m, n, k = (int(rng.integers(1, 401)) for _ in range(3))
        if case % 7 == 0:
            m, n, k = 128 * int(rng.integers(1, 4)), 96 * int(rng.integers(1, 4)), 32 * int(rng.integers(1, 9))  # exactly tiled
        ta, tb = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        pad_a, pad_b = int(rng.integers(0, 3)), int(rng.integers(0, 3))
        sa = (k, m) if ta else (m, k)
        sb = (n, k) if tb else (k, n)
        big_a = rng.uniform(-1, 1, (sa[0] + 2 * pad_a, sa[1])).astype(np.float32)
        big_b = rng.uniform(-1, 1, (sb[0] + 2 * pad_b, sb[1])).astype(np.float32)
        say("gemm random", case, (m, n, k), ta, tb, pad_a, pad_b)
        ad, ao = view_pair(ctx, big_a, lambda t: t.slice(0, pad_a, pad_a + sa[0]))
        bd, bo = view_pair(ctx, big_b, lambda t: t.slice(0, pad_b, pad_b + sb[0]))
        a64 = big_a[pad_a:pad_a + sa[0]].astype(np.float64)
        b64 = big_b[pad_b:pad_b + sb[0]].astype(np.float64)
        ref = (a64.T if ta else a64) @ (b64.T if tb else b64)
        y = V.gemm(ad, bd, ta, tb)
        yo = O.gemm(ao, bo, ta, tb)
        kind = case % 3
        if kind >= 1:
            bias = rng.uniform(-1, 1, (n,)).astype(np.float32)
            y, yo, ref = y + dev(ctx, bias), O.binary("add", yo, ht(bias).expand([m, n])), ref + bias
        if kind == 2:
            res = rng.uniform(-1, 1, (m, n)).astype(np.float32)
            y, yo, ref = nn.relu(y) + dev(ctx, res), O.binary("add", O.relu(yo), ht(res)), np.maximum(ref, 0) + res
        out = y.eval(ctx).numpy()
        close(out, ref, REL_GEMM, f"case {case} vs float64")
        close(out, yo.numpy(), REL_GEMM, f"case {case} vs oracle")


@pytest.mark.parametrize("m,k,n", [(128, 512, 10), (64, 768, 2), (1, 1, 1), (7, 1000, 16), (300, 65, 3), (5, 257, 13), (512, 129, 16), (513, 129, 16)])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_gemm_skinny_outputs(ctx, m, k, n, ta, tb):
    """Products with at most 16 output columns and at most 512 rows (classifier heads) run one wavefront per output row
    instead of MFMA tiles + split-K (513 rows: tiles again): all four transpose modes, with bias / ReLU / residual, against float64 and the oracle; the sum
    order is fixed, so the same call gives the same bits."""
    say("gemm skinny", (m, k, n), ta, tb)
    rng = np.random.default_rng(m * 3 + k + n)
    a = rng.uniform(-1, 1, (k, m) if ta else (m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (n, k) if tb else (k, n)).astype(np.float32)
    bias = rng.uniform(-1, 1, (n,)).astype(np.float32)
    res = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    ref64 = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
    n0 = ctx.launches
    y = V.gemm(dev(ctx, a), dev(ctx, b), ta, tb).eval(ctx).numpy()
    assert ctx.launches - n0 == 1
    close(y, ref64, REL_GEMM, "gemm vs float64")
    close(y, O.gemm(ht(a), ht(b), ta, tb).numpy(), REL_GEMM, "gemm vs oracle")
    y2 = (nn.relu(V.gemm(dev(ctx, a), dev(ctx, b), ta, tb) + dev(ctx, bias)) + dev(ctx, res)).eval(ctx).numpy()
    close(y2, np.maximum(ref64 + bias, 0) + res, REL_GEMM, "relu(gemm + bias) + residual vs float64")
    exact(y, V.gemm(dev(ctx, a), dev(ctx, b), ta, tb).eval(ctx).numpy(), "same call, same bits")


def test_gemm_batched_split_k(ctx_under):
    say("gemm_batched split-K")
    ctx = ctx_under(SAGE_GEMM_SPLITK="4")
    rng = np.random.default_rng(77)
    bt, m, k, n = 3, 37, 300, 44
    a = rng.uniform(-1, 1, (bt, m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (bt, k, n)).astype(np.float32)
    y = V.gemm_batched(dev(ctx, a), dev(ctx, b), False, False).eval(ctx).numpy()
    close(y, np.einsum("bmk,bkn->bmn", a.astype(np.float64), b.astype(np.float64)), REL_GEMM, "batched split")
    close(y, O.gemm_batched(ht(a), ht(b), False, False).numpy(), REL_GEMM, "vs oracle")


@pytest.mark.parametrize("split", [None, "3"])
def test_matmul_strided_residual_with_flattened_batch(ctx, ctx_under, split):
    """C has two batch axes [2,3,M,N]; the residual is [6,M,N] (batch axes flattened), [2,3,M,N] or a
    single [M,N]-per-batch view: all three address batch entry b0*3+b1 (straight through the C ABI)."""
    say("matmul_strided residual layouts", split)
    if split:
        ctx = ctx_under(SAGE_GEMM_SPLITK=split)
    lib = abi.lib()
    rng = np.random.default_rng(91)
    b0, b1, m, k, n = 2, 3, 40, 96, 36
    a = rng.uniform(-1, 1, (b0, b1, m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (b0, b1, k, n)).astype(np.float32)
    r = rng.uniform(-1, 1, (b0, b1, m, n)).astype(np.float32)
    ref = np.einsum("abmk,abkn->abmn", a.astype(np.float64), b.astype(np.float64)) + r
    ta, tb = S.Tensor.from_numpy(ctx, a), S.Tensor.from_numpy(ctx, b)
    for res_host in (r.reshape(b0 * b1, m, n), r):
        tr = S.Tensor.from_numpy(ctx, res_host)
        out = S.Tensor.uninit(ctx, [b0, b1, m, n])
        ac, bc, oc, rc_ = ta.c(), tb.c(), out.c(), tr.c()
        epi = abi.sg_gemm_epilogue(1.0, abi.ACT_NONE, abi.ACT_NONE, None, C.pointer(rc_))
        ctx.check(lib.sg_matmul_strided(ctx.handle, C.byref(ac), C.byref(bc), C.byref(oc), C.byref(epi)))
        close(out.numpy(), ref, REL_GEMM, f"residual rank {res_host.ndim}")


def test_gemm_offsets_and_ld(ctx):
    """ld = strides[0] and element offsets, as gemm.rs:208-217 passes them: slices of larger matrices."""
    say("gemm ld/offset")
    rng = np.random.default_rng(31)
    big_a = rng.uniform(-1, 1, (40, 90)).astype(np.float32)
    big_b = rng.uniform(-1, 1, (100, 50)).astype(np.float32)
    ad, ao = view_pair(ctx, big_a, lambda t: t.slice(0, 3, 36))
    bd, bo = view_pair(ctx, big_b, lambda t: t.slice(0, 10, 100))
    y = V.gemm(ad, bd).eval(ctx).numpy()
    close(y, big_a[3:36].astype(np.float64) @ big_b[10:100].astype(np.float64), REL_GEMM, "row slices (offset, default strides)")
    close(y, O.gemm(ao, bo).numpy(), REL_GEMM, "oracle")
    # a column window has strides != default: the reference organizes (copies) it first, gemm.rs:111
    ad, ao = view_pair(ctx, big_a, lambda t: t.slice(1, 5, 55))
    bd, bo = view_pair(ctx, big_b, lambda t: t.slice(0, 0, 50))
    close(V.gemm(ad, bd).eval(ctx).numpy(), O.gemm(ao, bo).numpy(), REL_GEMM, "column window")


@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_gemm_batched(ctx, ta, tb):
    say("gemm_batched", ta, tb)
    rng = np.random.default_rng(17)
    bt, m, k, n = 5, 37, 29, 41
    a = rng.uniform(-1, 1, (bt, k, m) if ta else (bt, m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (bt, n, k) if tb else (bt, k, n)).astype(np.float32)
    y = V.gemm_batched(dev(ctx, a), dev(ctx, b), ta, tb).eval(ctx).numpy()
    close(y, O.gemm_batched(ht(a), ht(b), ta, tb).numpy(), REL_GEMM, "gemm_batched")


def test_matmul_and_matmul_batched(ctx):
    """matmul (gemm.rs:30-51) on rank-3 x rank-2; matmul_batched (gemm.rs:53-104) on attention layouts,
    strided in place (fused) and through the reference's organize copies (unfused)."""
    rng = np.random.default_rng(19)
    x = rng.uniform(-1, 1, (3, 10, 24)).astype(np.float32)
    w = rng.uniform(-1, 1, (24, 16)).astype(np.float32)
    say("matmul [3,10,24] x [24,16]")
    close(dev(ctx, x).matmul(dev(ctx, w)).eval(ctx).numpy(), O.matmul(ht(x), ht(w)).numpy(), REL_GEMM, "matmul")
    n, l, h, d = 2, 20, 3, 8
    q = rng.uniform(-1, 1, (n, l, h * d)).astype(np.float32)
    k = rng.uniform(-1, 1, (n, l, h * d)).astype(np.float32)
    for fused in (True, False):
        V.set_fusion(fused)
        say("attention scores, fusion", fused)
        sep = lambda t: t.view([n, l, h, d]).transpose(2, 1)
        s_d = sep(dev(ctx, q)).matmul_batched(sep(dev(ctx, k)).transpose(-1, -2))
        s_o = O.matmul_batched(sep(ht(q)), sep(ht(k)).transpose(-1, -2))
        n0 = ctx.launches
        sd = s_d.eval(ctx).numpy()
        if fused:
            assert ctx.launches - n0 == 1  # no organize copies
        close(sd, s_o.numpy(), REL_GEMM, "QK^T")
        say("attention values + merge_heads, fusion", fused)
        p = rng.uniform(0, 1, (n, h, l, l)).astype(np.float32)
        av_d = dev(ctx, p).matmul_batched(sep(dev(ctx, k))).transpose(2, 1).view([n, l, h * d])
        av_o = O.matmul_batched(ht(p), sep(ht(k))).transpose(2, 1).view([n, l, h * d])
        n0 = ctx.launches
        avd = av_d.eval(ctx).numpy()
        if fused:
            assert ctx.launches - n0 == 1  # result written in merged layout, no copy
        close(avd, av_o.numpy(), REL_GEMM, "PV merged")


def test_gemm_epilogues(ctx):
    """Dense (+bias), Dense+ReLU, Dense+GELU, Dense+bias+residual, relu(conv+bias+x), scores/8."""
    rng = np.random.default_rng(23)
    x = rng.standard_normal((6, 11, 40)).astype(np.float32)
    w = (rng.standard_normal((40, 24)) * 0.2).astype(np.float32)
    b = rng.standard_normal((24,)).astype(np.float32)
    r = rng.standard_normal((6, 11, 24)).astype(np.float32)
    cases = {
        "bias": (lambda X, W, Bi, R: X.matmul(W) + Bi, lambda X, W, Bi, R: O.dense(X, W, Bi)),
        "bias_relu": (lambda X, W, Bi, R: nn.relu(X.matmul(W) + Bi), lambda X, W, Bi, R: O.relu(O.dense(X, W, Bi))),
        "bias_gelu": (lambda X, W, Bi, R: nn.gelu(X.matmul(W) + Bi),
                      lambda X, W, Bi, R: O.binary("mul", O.binary("mul", O.dense(X, W, Bi), 0.5),
                                                   O.binary("add", O.unary("erf", O.binary("div", O.dense(X, W, Bi), float(np.sqrt(np.float32(2))))), 1.0))),
        "bias_res": (lambda X, W, Bi, R: (X.matmul(W) + Bi) + R, lambda X, W, Bi, R: O.binary("add", O.dense(X, W, Bi), R)),
        "res_first": (lambda X, W, Bi, R: R + (X.matmul(W) + Bi), lambda X, W, Bi, R: O.binary("add", R, O.dense(X, W, Bi))),
        "relu_bias_res": (lambda X, W, Bi, R: nn.relu((X.matmul(W) + Bi) + R), lambda X, W, Bi, R: O.relu(O.binary("add", O.dense(X, W, Bi), R))),
        "scale": (lambda X, W, Bi, R: X.matmul(W) / 8.0, lambda X, W, Bi, R: O.binary("div", O.matmul(X, W), 8.0)),
    }
    for name, (fd, fo) in cases.items():
        say("epilogue", name)
        n0 = ctx.launches
        y = fd(dev(ctx, x), dev(ctx, w), dev(ctx, b), dev(ctx, r)).eval(ctx).numpy()
        assert ctx.launches - n0 == 1, f"{name}: expected one fused GEMM launch, got {ctx.launches - n0}"
        close(y, fo(ht(x), ht(w), ht(b), ht(r)).numpy(), REL_GEMM, name)
        V.set_fusion(False)
        yu = fd(dev(ctx, x), dev(ctx, w), dev(ctx, b), dev(ctx, r)).eval(ctx).numpy()
        V.set_fusion(True)
        close(y, yu, REL_GEMM, name + " vs unfused")
    say("shared GEMM output is not folded twice")
    X, W, Bi = dev(ctx, x), dev(ctx, w), dev(ctx, b)
    g = X.matmul(W)
    y1, y2 = S.evaluate(ctx, [g + Bi, g * 2.0])
    close(y2.numpy(), 2.0 * (y1.numpy() - b), REL_GEMM, "shared")


@pytest.mark.parametrize("with_res", [False, True])
def test_gemm_direct_write_out_with_special_bias_values(ctx, with_res):
    """Exactly tiled products without activation leave through the write-out that starts the accumulators at
    bias + residual (the bias joins through the matrix pipe): infinities, NaN and huge values in the bias stay in
    their own columns, everything else agrees with float64."""
    say("direct write-out, special bias values, residual", with_res)
    rng = np.random.default_rng(31)
    m, k, n = 256, 96, 192
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    bias = rng.uniform(-1, 1, (n,)).astype(np.float32)
    bias[[0, 33, 95, 96, 191]] = [np.inf, -np.inf, np.nan, -0.0, 3e38]
    res = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    lib = abi.lib()
    ta, tb, tbias, tres = (S.Tensor.from_numpy(ctx, x) for x in (a, b, bias, res))
    out = S.Tensor.uninit(ctx, [m, n])
    ac, bc, oc, biasc, resc = ta.c(), tb.c(), out.c(), tbias.c(), tres.c()
    epi = abi.sg_gemm_epilogue(1.0, abi.ACT_NONE, abi.ACT_NONE, C.pointer(biasc), C.pointer(resc) if with_res else None)
    ctx.check(lib.sg_gemm(ctx.handle, 0, 0, C.byref(ac), C.byref(bc), C.byref(oc), C.byref(epi)))
    name = C.create_string_buffer(128)
    lib.sg_gemm_last_kernel_name(ctx.handle, name, 128)
    assert b"false, false, true>" in name.value, f"expected an unguarded instantiation with the direct write-out, got {name.value}"
    got = out.numpy()
    with np.errstate(all="ignore"):
        want = a.astype(np.float64) @ b.astype(np.float64) + bias.astype(np.float64) + (res if with_res else 0.0)
    assert np.all(got[:, 0] == np.inf) and np.all(got[:, 33] == -np.inf) and np.all(np.isnan(got[:, 95]))
    assert np.all(np.isfinite(got[:, 191])) and np.allclose(got[:, 191], 3e38, rtol=1e-6)
    ok = np.ones(n, bool)
    ok[[0, 33, 95, 191]] = False
    close(got[:, ok], want[:, ok], REL_GEMM, "finite columns")


@pytest.mark.parametrize("m,n", [(128, 96), (256, 128), (100, 70)])
def test_gemm_gelu_epilogue_over_the_whole_range(ctx, m, n):
    """The product kernels' GELU (a table of cubic pieces of the normal distribution function in LDS) against float64
    0.5 x (1 + erf(x / sqrt 2)): over [-9, 9], at the table's nodes and ends, far outside it, on zeros, infinities and NaN.
    The pre-activations are exact: y = gelu(X . I), every product with one non-zero term."""
    import math
    say("gelu epilogue", m, n)
    rng = np.random.default_rng(41)
    vals = np.concatenate([np.linspace(-9, 9, 4001), -6 + np.arange(0, 385) / 32, [-6.0001, 5.99999, 6.0, 6.0001, -100, 100, -1e30, 1e30, 0.0, -0.0, 1e-30, -1e-30],
                           rng.standard_normal(4000) * 2]).astype(np.float32)
    x = np.resize(vals, m * n).reshape(m, n)
    lib = abi.lib()
    tx, teye, to = S.Tensor.from_numpy(ctx, x), S.Tensor.from_numpy(ctx, np.eye(n, dtype=np.float32)), S.Tensor.uninit(ctx, [m, n])
    xc, eyec, oc = tx.c(), teye.c(), to.c()
    epi = abi.sg_gemm_epilogue(1.0, abi.ACT_GELU_ERF, abi.ACT_NONE, None, None)
    ctx.check(lib.sg_gemm(ctx.handle, 0, 0, C.byref(xc), C.byref(eyec), C.byref(oc), C.byref(epi)))
    got = to.numpy()
    xf = x.astype(np.float64)
    want = 0.5 * xf * (1.0 + np.vectorize(math.erf)(xf / math.sqrt(2.0)))
    err = np.abs(got - want)
    bound = 6e-7 * np.maximum(1.0, np.abs(xf))
    worst = np.unravel_index(np.argmax(err - bound), err.shape)
    assert np.all(err <= bound), f"gelu({x[worst]}) = {got[worst]}, float64 {want[worst]}"
    # infinities and NaN arrive through the bias (as operands of the product they would spread over their rows)
    special = np.array([np.inf, -np.inf, np.nan, -0.0] + [0.0] * (n - 4), np.float32)
    tz, tbias = S.Tensor.from_numpy(ctx, np.zeros((m, n), np.float32)), S.Tensor.from_numpy(ctx, special)
    zc, biasc = tz.c(), tbias.c()
    epi = abi.sg_gemm_epilogue(1.0, abi.ACT_GELU_ERF, abi.ACT_NONE, C.pointer(biasc), None)
    ctx.check(lib.sg_gemm(ctx.handle, 0, 0, C.byref(zc), C.byref(eyec), C.byref(oc), C.byref(epi)))
    got = to.numpy()
    # (-inf times the 0 it approaches is NaN in the reference's 0.5 x (1 + erf) as well)
    assert np.all(got[:, 0] == np.inf) and np.all(np.isnan(got[:, 1])) and np.all(np.isnan(got[:, 2])), got[0, :4]
    assert np.all(got[:, 3:] == 0.0)


# ----------------------------------------------------------------------------- conv
IM2COL_CASES = [
    ((2, 28, 28, 1), 7, 2, 3, 1), ((2, 14, 14, 64), 3, 2, 1, 1), ((3, 7, 7, 64), 3, 1, 1, 1), ((2, 7, 7, 64), 1, 2, 0, 1),
    ((1, 5, 4, 3), [3, 2], 1, 0, 1), ((2, 9, 11, 6), [2, 3], [2, 1], [1, 2], [2, 1]), ((2, 1, 1, 512), 1, 1, 0, 1),
]


@pytest.mark.parametrize("case", range(len(IM2COL_CASES)))
def test_im2col(ctx, case):
    shape, ker, stride, pad, dil = IM2COL_CASES[case]
    say("im2col", shape, ker, stride, pad, dil)
    x = np.random.default_rng(case).standard_normal(shape).astype(np.float32)
    exact(V.im2col(dev(ctx, x), ker, stride, pad, dil).eval(ctx).numpy(), O.im2col(ht(x), ker, stride, pad, dil).numpy(), "im2col")


def test_conv_and_pools(ctx):
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(29)
    x = rng.standard_normal((2, 12, 10, 5)).astype(np.float32)
    f = (rng.standard_normal((3, 3, 5, 7)) * 0.3).astype(np.float32)
    b = rng.standard_normal((7,)).astype(np.float32)
    say("conv2d vs oracle and torch")
    from sage_amd.layers import Conv2d
    conv = Conv2d(5, 7, 3, 2, 1, 1)
    conv.weight.set(S.Tensor.from_numpy(ctx, f))
    conv.bias.set(S.Tensor.from_numpy(ctx, b))
    y = conv.pass_(dev(ctx, x)).eval(ctx).numpy()
    close(y, O.conv2d_layer(ht(x), ht(f), ht(b), 2, 1).numpy(), REL_GEMM, "conv oracle")
    t = F.conv2d(torch.from_numpy(x).permute(0, 3, 1, 2).double(), torch.from_numpy(f).permute(3, 2, 0, 1).double(),
                 torch.from_numpy(b).double(), stride=2, padding=1).permute(0, 2, 3, 1).numpy()
    close(y, t, REL_GEMM, "conv torch")
    say("max / avg pool")
    xp = np.abs(x)
    exact(V.max_pool_2d(dev(ctx, xp), 3, 2, 1, 1).eval(ctx).numpy(), O.max_pool_2d(ht(xp), 3, 2, 1, 1).numpy(), "max_pool")
    close(V.avg_pool_2d(dev(ctx, xp), 2, 2, 0, 1).eval(ctx).numpy(), O.avg_pool_2d(ht(xp), 2, 2, 0, 1).numpy(), REL_MAP, "avg_pool")


@pytest.mark.parametrize("geom", [((2, 5, 6, 4), (3, 3, 4, 4), 2, 1, 1), ((1, 7, 4, 8), (2, 3, 8, 8), [2, 1], [0, 1], [1, 2]),
                                  ((1, 7, 4, 8), (2, 3, 8, 8), [1, 2], [1, 0], [2, 2]), ((3, 4, 4, 6), (3, 3, 5, 6), 2, 0, 1), ((2, 6, 6, 16), (4, 4, 16, 16), 2, 1, 1)])
def test_conv_transpose_2d(ctx, geom):
    """conv_transpose_2d (conv.rs:98-140) = view -> matmul with the permuted filter -> col2im, onto the
    reference's output size (conv.rs:33-45, one less per side than the usual formula).  Against the oracle's
    composition where the reference defines a result (with two different dilations its col2im kernel takes tap
    indices from the wrong dilation and reads other taps' entries, conv.rs:463-465: the oracle refuses that
    geometry and the product returns the adjoint), and, where the filter's two channel extents are equal (the only
    case in which the reference's view of the filter is a transposition), against torch's conv_transpose2d cropped
    to that size."""
    import torch
    import torch.nn.functional as F
    xs, fs, stride, pad, dil = geom
    say("conv_transpose_2d", geom)
    rng = np.random.default_rng(sum(xs) + sum(fs))
    x = rng.standard_normal(xs).astype(np.float32)
    f = (rng.standard_normal(fs) * 0.3).astype(np.float32)
    y = V.conv_transpose_2d(dev(ctx, x), dev(ctx, f), stride, pad, dil).eval(ctx).numpy()
    pr = lambda v: [v, v] if isinstance(v, int) else list(v)  # [w, h] pairs
    st, pd, dl = pr(stride), pr(pad), pr(dil)
    if dl[0] == dl[1]:
        yo = O.conv_transpose_2d(ht(x), ht(f), stride, pad, dil).numpy()
        assert y.shape == yo.shape
        close(y, yo, REL_GEMM, "conv_transpose_2d vs oracle")
    else:
        assert fs[2] == fs[3], "a geometry the oracle refuses needs the torch comparison"
        with pytest.raises(RuntimeError, match="or_col2im"):
            O.conv_transpose_2d(ht(x), ht(f), stride, pad, dil)
    if fs[2] == fs[3]:
        # torch's weight is [C_in, C_out, KH, KW]; the reference contracts x's channels with filter axis 2
        t = F.conv_transpose2d(torch.from_numpy(x).permute(0, 3, 1, 2).double(), torch.from_numpy(f).permute(2, 3, 0, 1).double(),
                               stride=(st[1], st[0]), padding=(pd[1], pd[0]), dilation=(dl[1], dl[0])).permute(0, 2, 3, 1).numpy()
        assert t.shape[1] == y.shape[1] + 1 and t.shape[2] == y.shape[2] + 1
        close(y, t[:, :y.shape[1], :y.shape[2], :], REL_GEMM, "conv_transpose_2d vs torch")
    with pytest.raises(abi.ShapeError):
        V.conv_transpose_2d(dev(ctx, x), dev(ctx, f[:, :, :, :-1].copy()), stride, pad, dil)


CONV_CASES = [
    # (n, h, w, c, kh, kw, oc, stride [w,h], pad [w,h], dil [w,h])
    (2, 12, 10, 5, 3, 3, 7, [2, 2], [1, 1], [1, 1]),      # channels not a multiple of 4: scalar taps
    (3, 28, 28, 1, 7, 7, 64, [2, 2], [3, 3], [1, 1]),     # the first ResNet convolution: one channel, K = 49
    (4, 14, 14, 64, 3, 3, 64, [1, 1], [1, 1], [1, 1]),    # 16-byte channel loads, exactly tiled N
    (2, 9, 11, 8, 3, 2, 12, [1, 2], [2, 0], [2, 1]),      # rectangular kernel, mixed stride/padding, dilation
    (2, 7, 7, 128, 1, 1, 256, [2, 2], [0, 0], [1, 1]),    # 1x1 stride-2 downsample
    (16, 4, 4, 256, 3, 3, 256, [1, 1], [1, 1], [1, 1]),   # few output tiles and K = 2304: split-K
    (1, 6, 6, 4, 3, 3, 8, [1, 1], [1, 1], [0, 0]),        # dilation 0 (every tap reads the window's corner, as the reference would)
    # exactly tiled outputs with C % 16 == 0: the unguarded instantiation, A fetched with buffer loads, border taps masked
    (4, 8, 8, 64, 3, 3, 64, [1, 1], [1, 1], [1, 1]),      # M = 256, K = 576
    (4, 8, 8, 32, 3, 3, 128, [2, 2], [1, 1], [1, 1]),     # stride 2: M = 64, K = 288
    (2, 16, 8, 16, 7, 7, 64, [1, 1], [3, 3], [1, 1]),     # 49 taps, M = 256, K = 784 (not a multiple of 32: guarded after all)
    (2, 16, 8, 32, 5, 3, 64, [1, 1], [2, 1], [2, 1]),     # 15 taps, dilation 2 across the width, M = 256, K = 480
    (8, 4, 4, 128, 1, 1, 64, [2, 2], [0, 0], [1, 1]),     # 1x1 stride 2 downsample: M = 32 ... guarded; and
    (32, 4, 4, 128, 1, 1, 64, [2, 2], [0, 0], [1, 1]),    # the same at M = 128: unguarded
    (64, 2, 2, 256, 3, 3, 256, [1, 1], [1, 1], [1, 1]),   # M = 256, K = 2304: unguarded and split-K
    # dilation and padding larger than the image, one image: exactly tiled (M = 64, K = 288, C % 16 == 0), but the last taps'
    # displacement lies beyond the image plus its lead, so the host must choose the guarded loads
    (1, 8, 8, 32, 3, 3, 64, [1, 1], [9, 9], [9, 9]),
    # taps that are padding for every output pixel are left out of the product when the rest of the filter is one block:
    (8, 1, 1, 32, 3, 3, 64, [1, 1], [1, 1], [1, 1]),      # 1x1 image, 3x3 window: the centre tap alone (K 288 -> 32)
    (64, 1, 1, 64, 3, 3, 64, [1, 1], [1, 1], [1, 1]),     # the same exactly tiled (M = 64): unguarded
    (4, 2, 6, 16, 3, 3, 32, [1, 2], [1, 1], [1, 1]),      # 2 rows, stride 2 down: tap rows 1..2 (whole rows of the filter)
    (2, 1, 5, 8, 3, 3, 16, [1, 1], [1, 1], [1, 1]),       # 1 row: the middle row of taps
    (4, 2, 2, 16, 3, 3, 32, [2, 2], [1, 1], [1, 1]),      # 2x2 -> 1x1 with stride 2: taps {1,2} x {1,2}, not one block: all nine walked
    (3, 1, 1, 5, 5, 5, 7, [1, 1], [2, 2], [1, 1]),        # 5x5 window over a 1x1 image, scalar loads
]


@pytest.mark.parametrize("case", CONV_CASES, ids=[f"c{i}" for i in range(len(CONV_CASES))])
def test_conv2d_without_column_matrix(ctx, monkeypatch, case):
    """sg_conv2d reads the GEMM's A operand from the image through the im2col window arithmetic.  It must
    equal the oracle's im2col + gemm (conv.rs:61-96) within the GEMM tolerance, and the explicit
    sg_im2col + sg_gemm path bit for bit where both split K the same way (same tiles, same k order; between
    K = 512 and 1024 the guarded image-addressed product is split and the plain one is not), with and without bias / ReLU / residual."""
    n, h, w, c, kh, kw, oc, stride, pad, dil = case
    say("conv2d", case)
    rng = np.random.default_rng(n * 100 + c)
    x = rng.standard_normal((n, h, w, c)).astype(np.float32)
    f = (rng.standard_normal((kh, kw, c, oc)) * 0.2).astype(np.float32)
    bias = rng.standard_normal((oc,)).astype(np.float32)

    def build(with_epilogue):
        y = V.conv_2d(dev(ctx, x), dev(ctx, f), stride, pad, dil)
        if with_epilogue:
            y = nn.relu(y + dev(ctx, bias)) + dev(ctx, res)
        return y

    yo = O.conv_2d(ht(x), ht(f), stride, pad, dil)
    res = rng.standard_normal(tuple(yo.extents)).astype(np.float32)
    for with_epilogue in (False, True):
        n0 = ctx.launches
        y_fused = build(with_epilogue).eval(ctx).numpy()
        fused_launches = ctx.launches - n0
        monkeypatch.setenv("SAGE_FUSE_CONV", "0")
        y_explicit = build(with_epilogue).eval(ctx).numpy()
        monkeypatch.delenv("SAGE_FUSE_CONV")
        ref = yo.numpy()
        if with_epilogue:
            ref = O.binary("add", O.relu(O.binary("add", yo, ht(bias))), ht(res)).numpy()
        close(y_fused, ref, REL_GEMM, "conv2d vs oracle")
        if 512 <= kh * kw * c < 1024 or oc <= 16:  # (a product with at most 16 columns over an existing column matrix is not an MFMA product)
            close(y_fused, y_explicit, REL_GEMM, "conv2d vs im2col + gemm")
        else:
            exact(y_fused, y_explicit, "conv2d vs im2col + gemm")
        assert fused_launches <= (2 if with_epilogue else 1), fused_launches


def test_product_over_another_factorisation_of_the_column_tensor_is_not_a_convolution(ctx):
    """A product whose operands are OTHER 2-D views of an im2col tensor and of a rank-4 [kh,kw,c,*] filter is a
    different contraction than conv_2d: it must run as im2col + gemm (two launches), not be handed to sg_conv2d."""
    say("gemm over a re-factored column tensor")
    rng = np.random.default_rng(5)
    x = rng.standard_normal((1, 4, 4, 2)).astype(np.float32)
    f = rng.standard_normal((2, 2, 2, 6)).astype(np.float32)
    col = V.im2col(dev(ctx, x), 2, 1, 0, 1)                      # [1,3,3,2,2,2] = 72 elements
    n0 = ctx.launches
    y = V.gemm(col.view([18, 4]), dev(ctx, f).view([4, 12]), False, False).eval(ctx).numpy()
    assert ctx.launches - n0 == 2
    colo = O.im2col(ht(x), [2, 2], [1, 1], [0, 0], [1, 1]).numpy().reshape(18, 4)
    close(y, colo.astype(np.float64) @ f.reshape(4, 12).astype(np.float64), REL_GEMM, "re-factored product")
    # the true convolution over the same operands is one launch
    n0 = ctx.launches
    yc = V.conv_2d(dev(ctx, x), dev(ctx, f), 1, 0, 1).eval(ctx).numpy()
    assert ctx.launches - n0 == 1
    close(yc.reshape(9, 6), O.im2col(ht(x), [2, 2], [1, 1], [0, 0], [1, 1]).numpy().reshape(9, 8).astype(np.float64) @ f.reshape(8, 6).astype(np.float64), REL_GEMM, "conv_2d")


@pytest.mark.parametrize("geom", [((2, 12, 10, 8), 3, 2, 1, 1), ((3, 14, 14, 64), 3, 2, 1, 1), ((2, 9, 7, 5), [2, 3], [1, 2], [1, 0], [2, 1]),
                                  ((4, 7, 7, 16), 7, 7, 0, 1), ((1, 6, 6, 3), 2, 2, 0, 1)])
def test_pooling_without_column_tensor(ctx, monkeypatch, geom):
    """max_pool_2d / avg_pool_2d (conv.rs:143-165) as one window kernel: bit-exact against the oracle's
    im2col + reduce for max (negative inputs included: the reference's accumulator starts at 0 and padding
    pixels are zeros), within the reduction tolerance for the mean, and equal to the two-launch path."""
    shape, ker, stride, pad, dil = geom
    say("pool2d", geom)
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal(shape).astype(np.float32)
    n0 = ctx.launches
    ymax = V.max_pool_2d(dev(ctx, x), ker, stride, pad, dil).eval(ctx).numpy()
    assert ctx.launches - n0 == 1
    exact(ymax, O.max_pool_2d(ht(x), ker, stride, pad, dil).numpy(), "max_pool vs oracle")
    yavg = V.avg_pool_2d(dev(ctx, x), ker, stride, pad, dil).eval(ctx).numpy()
    close(yavg, O.avg_pool_2d(ht(x), ker, stride, pad, dil).numpy(), REL_MAP, "avg_pool vs oracle")
    ymin = V.im2col(dev(ctx, x), ker, stride, pad, dil).min([3, 4], True).eval(ctx).numpy()
    monkeypatch.setenv("SAGE_FUSE_CONV", "0")
    exact(ymax, V.max_pool_2d(dev(ctx, x), ker, stride, pad, dil).eval(ctx).numpy(), "max_pool vs im2col + reduce")
    close(yavg, V.avg_pool_2d(dev(ctx, x), ker, stride, pad, dil).eval(ctx).numpy(), REL_MAP, "avg_pool vs im2col + reduce")
    exact(ymin, V.im2col(dev(ctx, x), ker, stride, pad, dil).min([3, 4], True).eval(ctx).numpy(), "min with preserved axes")


def test_conv2d_abi_errors(ctx):
    say("conv2d error behaviour")
    lib = abi.lib()
    x = S.Tensor.from_numpy(ctx, np.zeros((1, 5, 5, 4), np.float32))
    f = S.Tensor.from_numpy(ctx, np.zeros((3, 3, 4, 8), np.float32))
    f_bad = S.Tensor.from_numpy(ctx, np.zeros((3, 3, 5, 8), np.float32))
    out = S.Tensor.uninit(ctx, [1, 5, 5, 8])
    out_bad = S.Tensor.uninit(ctx, [1, 4, 5, 8])
    arr = lambda a, b: (C.c_int32 * 2)(a, b)
    xc, fc, fbc, oc, obc = x.c(), f.c(), f_bad.c(), out.c(), out_bad.c()
    assert lib.sg_conv2d(ctx.handle, C.byref(xc), C.byref(fc), C.byref(oc), arr(1, 1), arr(1, 1), arr(1, 1), None) == abi.OK
    assert lib.sg_conv2d(ctx.handle, C.byref(xc), C.byref(fbc), C.byref(oc), arr(1, 1), arr(1, 1), arr(1, 1), None) == abi.ERR_SHAPE  # conv.rs:86
    assert lib.sg_conv2d(ctx.handle, C.byref(xc), C.byref(fc), C.byref(obc), arr(1, 1), arr(1, 1), arr(1, 1), None) == abi.ERR_SHAPE
    assert lib.sg_conv2d(ctx.handle, C.byref(xc), C.byref(fc), C.byref(oc), arr(0, 1), arr(1, 1), arr(1, 1), None) == abi.ERR_ARG
    big = S.Tensor.from_numpy(ctx, np.zeros((9, 9, 4, 8), np.float32))
    bc = big.c()
    assert lib.sg_conv2d(ctx.handle, C.byref(xc), C.byref(bc), C.byref(oc), arr(1, 1), arr(0, 0), arr(1, 1), None) == abi.ERR_SHAPE  # kernel larger than image
    ctx.sync()


def test_last_product_kernel_name(ctx):
    """sg_gemm_last_kernel_name names the instantiation the most recent product launched: tile, operand layouts,
    guarded loads and image addressing, as a kernel trace prints it."""
    say("last product kernel name")
    lib = abi.lib()
    arr = lambda a, b: (C.c_int32 * 2)(a, b)

    def last():
        buf = C.create_string_buffer(128)
        ctx.check(lib.sg_gemm_last_kernel_name(ctx.handle, buf, 128))
        return buf.value.decode()

    rng = np.random.default_rng(3)
    a, b = dev(ctx, rng.standard_normal((256, 64)).astype(np.float32)), dev(ctx, rng.standard_normal((64, 128)).astype(np.float32))
    a.matmul(b).eval(ctx)
    assert last() == "gemm_mfma_kernel<64, 64, 2, true, true, false, false, true>", last()   # unguarded, plain product: the direct write-out
    dev(ctx, rng.standard_normal((70, 33)).astype(np.float32)).matmul(dev(ctx, rng.standard_normal((33, 19)).astype(np.float32))).eval(ctx)
    assert ", true, true, true, false, false>" in last(), last()   # guarded loads
    dev(ctx, rng.standard_normal((70, 33)).astype(np.float32)).matmul(dev(ctx, rng.standard_normal((33, 9)).astype(np.float32))).eval(ctx)
    assert last() == "gemm_skinny_kernel<16>", last()   # at most 16 output columns: a wavefront per output row
    dev(ctx, rng.standard_normal((70, 33)).astype(np.float32)).matmul(dev(ctx, rng.standard_normal((33, 2)).astype(np.float32))).eval(ctx)
    assert last() == "gemm_skinny_kernel<4>", last()
    for c, want in ((64, "gemm_mfma_kernel<64, 64, 2, true, true, false, true, true>"), (5, "true, true, true, true, false>")):
        x = S.Tensor.from_numpy(ctx, rng.standard_normal((4, 8, 8, c)).astype(np.float32))
        f = S.Tensor.from_numpy(ctx, rng.standard_normal((3, 3, c, 64)).astype(np.float32))
        out = S.Tensor.uninit(ctx, [4, 8, 8, 64])
        xc, fc, oc = x.c(), f.c(), out.c()
        ctx.check(lib.sg_conv2d(ctx.handle, C.byref(xc), C.byref(fc), C.byref(oc), arr(1, 1), arr(1, 1), arr(1, 1), None))
        assert last().endswith(want), last()   # image-addressed: unguarded with 16-channel slabs, guarded otherwise
    assert lib.sg_gemm_last_kernel_name(ctx.handle, None, 128) == abi.ERR_ARG
    ctx.sync()


# ----------------------------------------------------------------------------- fused row operators
@pytest.mark.parametrize("shape", [(64, 128), (5, 1000), (3, 4, 16, 16), (9, 1024), (2, 2052), (7, 10)])
def test_softmax_fused_vs_composed_vs_oracle(ctx, shape):
    say("softmax", shape)
    rng = np.random.default_rng(len(shape))
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    x[0] -= 20.0  # an all-negative row: the reference's zero-initialised max shows here
    ax = len(shape) - 1
    yf = nn.softmax(dev(ctx, x), ax).eval(ctx).numpy()
    V.set_fusion(False)
    yc = nn.softmax(dev(ctx, x), ax).eval(ctx).numpy()
    yo = O.softmax(ht(x), ax).numpy()
    close(yf, yo, REL_MAP, "fused vs oracle")
    close(yc, yo, REL_MAP, "composed vs oracle")
    close(yf.sum(-1), np.ones(shape[:-1]), 1e-5, "rows sum to 1")


def test_softmax_with_mask_addend(ctx):
    say("softmax(scores/8 + mask)")
    rng = np.random.default_rng(41)
    n, h, l = 3, 2, 32
    s = rng.standard_normal((n, h, l, l)).astype(np.float32) * 4
    m = (rng.uniform(0, 1, (n, l)) > 0.3).astype(np.float32)
    m[:, 0] = 1.0

    def dev_expr():
        md = (-dev(ctx, m).view([n, 1, 1, l]) + 1.0) * -1e5
        return nn.softmax(dev(ctx, s) / 8.0 + md, 3)

    mo = O.binary("mul", O.binary("add", O.unary("neg", ht(m).view([n, 1, 1, l])), 1.0), -1e5)
    yo = O.softmax(O.binary("add", O.binary("div", ht(s), 8.0), mo), 3).numpy()
    close(dev_expr().eval(ctx).numpy(), yo, REL_MAP, "fused")
    V.set_fusion(False)
    close(dev_expr().eval(ctx).numpy(), yo, REL_MAP, "composed")


def _attention_f64(q, k, v, mask_add, scale):
    s = np.einsum("...qd,...kd->...qk", q.astype(np.float64), k.astype(np.float64)) * scale
    if mask_add is not None:
        s = s + mask_add
    e = np.exp(s - np.maximum(s.max(-1, keepdims=True), 0.0))
    return np.einsum("...qk,...kd->...qd", e / e.sum(-1, keepdims=True), v.astype(np.float64))


@pytest.mark.parametrize("n,h,lq,lk,d", [(2, 3, 128, 128, 64), (1, 2, 70, 70, 64), (2, 2, 33, 200, 32), (1, 1, 1, 5, 64), (3, 12, 256, 256, 64)])
@pytest.mark.parametrize("masked", [False, True])
def test_attention_fused_vs_composed_vs_oracle(ctx, n, h, lq, lk, d, masked):
    """softmax(q.k^T / sqrt(d) + mask) . v on the separate_heads views of bert.rs:282-291, merged back as
    bert.rs:293-302: one launch when fused; equal to the operator-by-operator result and the oracle."""
    say("attention", n, h, lq, lk, d, masked)
    rng = np.random.default_rng(n * 1000 + lq + lk + d)
    e = h * d
    qa, ka, va = (rng.standard_normal((n, l_, e)).astype(np.float32) for l_ in (lq, lk, lk))
    m = (rng.uniform(0, 1, (n, lk)) > 0.3).astype(np.float32)
    m[:, 0] = 1.0
    scale = float(np.sqrt(np.float32(d)))

    def heads(f, l_):
        return f.view([n, l_, h, d]).transpose(2, 1)

    def expr(mk):
        q, k, v = heads(mk(qa), lq), heads(mk(ka), lk), heads(mk(va), lk)
        att = q.matmul_batched(k.transpose(-1, -2))
        att = att / scale if d == 64 else att * (1.0 / scale)  # a division folds only when exact (power of two)
        if masked:
            att = att + (-mk(m).view([n, 1, 1, lk]) + 1.0) * -1e5
        return att, v

    att, v = expr(lambda a: dev(ctx, a))
    n0 = ctx.launches
    out = nn.softmax(att, 3).matmul_batched(v).transpose(2, 1)
    yf = out.view([n, lq, e]).eval(ctx).numpy()
    fused_launches = ctx.launches - n0
    V.set_fusion(False)
    att, v = expr(lambda a: dev(ctx, a))
    yc = nn.softmax(att, 3).matmul_batched(v).transpose(2, 1).view([n, lq, e]).eval(ctx).numpy()
    qh, kh, vh = (a.reshape(n, l_, h, d).transpose(0, 2, 1, 3) for a, l_ in ((qa, lq), (ka, lk), (va, lk)))
    madd = ((1.0 - m.astype(np.float64)) * -1e5)[:, None, None, :] if masked else None
    ref = _attention_f64(qh, kh, vh, madd, 1.0 / scale).transpose(0, 2, 1, 3).reshape(n, lq, e)
    close(yf, ref, REL_GEMM, "fused vs float64")
    close(yc, ref, REL_GEMM, "composed vs float64")
    close(yf, yc, REL_GEMM, "fused vs composed")
    assert fused_launches == (2 if masked else 1), fused_launches  # the mask expression + the attention kernel


@pytest.mark.parametrize("split", ["0", "1"])
@pytest.mark.parametrize("n,h,lq,lk,d", [(2, 3, 128, 128, 64), (1, 2, 70, 200, 64), (2, 2, 33, 31, 32), (1, 1, 64, 300, 64)])
def test_attention_key_split_variant_matches(ctx_under, split, n, h, lq, lk, d):
    """The kernel that gives the two 32-key halves of every key block to different wavefronts and merges their
    online-softmax states, forced on and off: both agree with float64 attention (ragged key counts leave one half
    partly or wholly past the end)."""
    say("attention key split", split, (n, h, lq, lk, d))
    ctx = ctx_under(SAGE_ATTENTION_SPLIT=split)
    lib = abi.lib()
    rng = np.random.default_rng(lq * 7 + lk)
    q, k, v = (rng.standard_normal((n, h, l, d)).astype(np.float32) for l in (lq, lk, lk))
    mask = (rng.uniform(size=(n, 1, 1, lk)) < 0.8).astype(np.float32)
    add = ((1.0 - mask) * -1e5).astype(np.float32)
    tq, tk, tv, ta = (S.Tensor.from_numpy(ctx, a) for a in (q, k, v, add))
    out = S.Tensor.uninit(ctx, [n, h, lq, d])
    from sage_amd.shape import Shape
    tadd = ta.with_shape(Shape([n, h, lq, lk], [lk, 0, 0, 1], 0))
    qc, kc, vc, ac, oc = tq.c(), tk.c(), tv.c(), tadd.c(), out.c()
    scale = 1.0 / np.sqrt(np.float32(d))
    ctx.check(lib.sg_attention(ctx.handle, C.byref(qc), C.byref(kc), C.byref(vc), C.byref(ac), C.c_float(scale), C.byref(oc)))
    s = np.einsum("nhqd,nhkd->nhqk", q.astype(np.float64), k.astype(np.float64)) * float(scale) + add
    s -= np.maximum(s.max(-1, keepdims=True), 0.0)
    p_ = np.exp(s)
    ref = np.einsum("nhqk,nhkd->nhqd", p_ / p_.sum(-1, keepdims=True), v.astype(np.float64))
    close(out.numpy(), ref, REL_GEMM, "attention vs float64")


@pytest.mark.parametrize("split", ["0", "1"])
def test_attention_unaligned_operands(ctx_under, split):
    """Operands that are views at an odd element offset with a row stride of d + 1: no 16-byte access is legal,
    the instantiation with scalar loads and stores runs; same result as float64 attention, and the padding
    elements between the output rows stay untouched."""
    say("attention on unaligned views, split", split)
    ctx = ctx_under(SAGE_ATTENTION_SPLIT=split)
    lib = abi.lib()
    from sage_amd.shape import Shape
    n, h, lq, lk, d = 2, 3, 70, 100, 64
    rng = np.random.default_rng(77)
    ld = d + 1

    def padded(l):
        buf = rng.standard_normal(1 + n * h * l * ld).astype(np.float32)
        view = buf[1:].reshape(n, h, l, ld)[..., :d]
        return buf, view

    (bq, q), (bk, k), (bv, v) = padded(lq), padded(lk), padded(lk)
    bo = np.full(1 + n * h * lq * ld, 7.0, np.float32)
    tensors = [S.Tensor.from_numpy(ctx, b) for b in (bq, bk, bv, bo)]
    shapes = [Shape([n, h, l, d], [h * l * ld, l * ld, ld, 1], 1) for l in (lq, lk, lk, lq)]
    qc, kc, vc, oc = (t.with_shape(sh).c() for t, sh in zip(tensors, shapes))
    scale = 1.0 / np.sqrt(np.float32(d))
    ctx.check(lib.sg_attention(ctx.handle, C.byref(qc), C.byref(kc), C.byref(vc), None, C.c_float(scale), C.byref(oc)))
    s = np.einsum("nhqd,nhkd->nhqk", q.astype(np.float64), k.astype(np.float64)) * float(scale)
    s -= np.maximum(s.max(-1, keepdims=True), 0.0)
    p_ = np.exp(s)
    ref = np.einsum("nhqk,nhkd->nhqd", p_ / p_.sum(-1, keepdims=True), v.astype(np.float64))
    got = tensors[3].numpy()
    close(got[1:].reshape(n, h, lq, ld)[..., :d], ref, REL_GEMM, "attention on unaligned views vs float64")
    assert got[0] == 7.0 and np.all(got[1:].reshape(n, h, lq, ld)[..., d] == 7.0)


def test_attention_fully_masked_row_is_reference_nan(ctx):
    """Every key masked by -1e5: the reference's softmax shifts by max(0, row max) = 0, every exp underflows
    and the row is 0/0.  The fused kernel keeps that behaviour instead of a uniform row."""
    say("attention fully masked")
    rng = np.random.default_rng(5)
    n, h, l, d = 2, 2, 64, 64
    qa, ka, va = (rng.standard_normal((n, l, h * d)).astype(np.float32) for _ in range(3))
    m = np.ones((n, l), np.float32)
    m[1, :] = 0.0

    def run():
        hd = lambda a: dev(ctx, a).view([n, l, h, d]).transpose(2, 1)
        att = hd(qa).matmul_batched(hd(ka).transpose(-1, -2)) / 8.0 + (-dev(ctx, m).view([n, 1, 1, l]) + 1.0) * -1e5
        return nn.softmax(att, 3).matmul_batched(hd(va)).eval(ctx).numpy()

    yf = run()
    V.set_fusion(False)
    yc = run()
    assert np.isnan(yf[1]).all() and np.isnan(yc[1]).all()
    close(yf[0], yc[0], REL_GEMM, "unmasked batch")


def test_attention_abi_errors(ctx):
    say("attention errors")
    q = S.Tensor.uninit(ctx, [2, 16, 48])
    with pytest.raises(abi.ShapeError):
        qc = q.c()
        ctx.check(ctx._lib.sg_attention(ctx.handle, C.byref(qc), C.byref(qc), C.byref(qc), None, C.c_float(1.0), C.byref(qc)))


@pytest.mark.parametrize("shape", [(5, 10), (512, 1024), (37, 1000), (16, 4096)])
def test_softmax_cross_entropy(ctx, shape):
    say("softmax_cross_entropy", shape)
    rng = np.random.default_rng(shape[0])
    x = rng.standard_normal(shape).astype(np.float32)
    lab = rng.integers(0, shape[1], (shape[0], 1)).astype(np.int32)
    yf = nn.softmax_cross_entropy(dev(ctx, x), dev(ctx, lab)).eval(ctx).numpy()
    V.set_fusion(False)
    yc = nn.softmax_cross_entropy(dev(ctx, x), dev(ctx, lab)).eval(ctx).numpy()
    yo = O.softmax_cross_entropy(ht(x), ht(lab.view(np.uint32).astype(np.uint32))).numpy()
    x64 = x.astype(np.float64)
    ref = -(x64[np.arange(shape[0]), lab[:, 0]] - np.log(np.exp(x64).sum(1)))
    for name, y in (("fused", yf), ("composed", yc), ("oracle", yo)):
        close(y, ref, REL_MAP, name + " vs float64")
    close(yf, yo, REL_MAP, "fused vs oracle")


def test_softmax_cross_entropy_rows_far_below_zero(ctx):
    """The shift is max(0, row max) (reduce.rs:282), so a row entirely below -87 sums terms under 2^-126:
    the fused kernel keeps them (denormal) like the composition and the oracle, it does not flush the sum
    to zero and the loss to infinity.  Rows partly below that limit and ordinary rows ride along."""
    say("softmax_cross_entropy far below zero")
    rng = np.random.default_rng(11)
    x = rng.standard_normal((64, 1024)).astype(np.float32)
    x[:16] = rng.uniform(-101.0, -89.0, (16, 1024)).astype(np.float32)     # every term denormal
    x[16:32] = rng.uniform(-95.0, -80.0, (16, 1024)).astype(np.float32)    # denormal and normal terms mixed
    x[32:40] -= 60.0
    lab = rng.integers(0, 1024, (64, 1)).astype(np.int32)
    yf = nn.softmax_cross_entropy(dev(ctx, x), dev(ctx, lab)).eval(ctx).numpy()
    yo = O.softmax_cross_entropy(ht(x), ht(lab.view(np.uint32))).numpy()
    assert np.all(np.isfinite(yo)) and np.all(np.isfinite(yf))
    x64 = x.astype(np.float64)
    ref = -(x64[np.arange(64), lab[:, 0]] - np.log(np.exp(x64).sum(1)))
    # denormal terms carry fewer bits: the all-denormal rows agree to 1e-2 absolute on losses near 10, the rest to REL_MAP
    assert np.max(np.abs(yf[:16] - yo[:16])) < 1e-2 and np.max(np.abs(yf[:16] - ref[:16])) < 0.1
    close(yf[16:], yo[16:], REL_MAP, "fused vs oracle")
    close(yf[16:], ref[16:], REL_MAP, "fused vs float64")


def test_softmax_rows_far_below_zero(ctx):
    """The same for the softmax row kernel, whose exponentials come from the hardware exp2 (results under 2^-126
    flushed to zero): a row entirely below -87 keeps the shift 0 (reduce.rs:282), every term is denormal, and the
    kernel redoes the row with the exact routine instead of dividing zero by zero.  Mixed and ordinary rows and a
    row with a masked half (the attention mask's -1e5) ride along; every row still sums to one."""
    say("softmax far below zero")
    rng = np.random.default_rng(12)
    x = rng.standard_normal((48, 128)).astype(np.float32)
    x[:16] = rng.uniform(-101.0, -89.0, (16, 128)).astype(np.float32)     # every term denormal
    x[16:32] = rng.uniform(-95.0, -80.0, (16, 128)).astype(np.float32)    # denormal and normal terms mixed
    add = np.zeros((48, 128), np.float32)
    add[40:, 64:] = -1e5
    yf = nn.softmax(dev(ctx, x) + dev(ctx, add), 1).eval(ctx).numpy()
    yo = O.softmax(O.binary("add", ht(x), ht(add)), [1]).numpy()
    x64 = (x + add).astype(np.float64)
    e = np.exp(x64 - np.maximum(x64.max(1, keepdims=True), 0.0))
    ref = e / e.sum(1, keepdims=True)
    assert np.all(np.isfinite(yf)) and np.all(np.isfinite(yo))
    assert np.max(np.abs(yf[:16] - ref[:16])) < 2e-3 and np.max(np.abs(yf[:16] - yo[:16])) < 2e-3   # few bits in denormal terms
    close(yf[16:], yo[16:], REL_MAP, "fused vs oracle")
    close(yf[16:], ref[16:], REL_MAP, "fused vs float64")
    close(yf.sum(1), np.ones(48), 1e-2, "rows sum to one")
    assert np.all(yf[40:, 64:] == 0.0)


@pytest.mark.parametrize("shape,per_feature", [((8, 16, 768), False), ((8, 16, 768), True), ((5, 100), False), ((3, 2050), True), ((64, 64), True)])
def test_layer_norm(ctx, shape, per_feature):
    say("layer_norm", shape, per_feature)
    rng = np.random.default_rng(shape[-1])
    x = (rng.standard_normal(shape) * 2 + 0.5).astype(np.float32)
    n = shape[-1] if per_feature else 1
    g = rng.uniform(0.5, 1.5, (n,)).astype(np.float32)
    b = rng.standard_normal((n,)).astype(np.float32)
    ax = len(shape) - 1
    yf = nn.layer_norm(dev(ctx, x), ax, dev(ctx, g), dev(ctx, b), 1e-5).eval(ctx).numpy()
    V.set_fusion(False)
    yc = nn.layer_norm(dev(ctx, x), ax, dev(ctx, g), dev(ctx, b), 1e-5).eval(ctx).numpy()
    yo = O.layer_norm(ht(x), ax, ht(g), ht(b), 1e-5).numpy()
    x64 = x.astype(np.float64)
    ref = (x64 - x64.mean(-1, keepdims=True)) / np.sqrt(x64.var(-1, keepdims=True) + 1e-5) * g + b
    close(yf, ref, 5e-4, "fused vs float64")
    close(yc, ref, 5e-4, "composed vs float64")
    close(yo, ref, 5e-4, "oracle vs float64")
    close(yf, yo, 5e-4, "fused vs oracle")


ROW_LENGTHS = [1, 3, 4, 7, 16, 17, 32, 36, 64, 68, 100, 128, 132, 200, 256, 260, 384, 512, 516, 768, 1000, 1024, 1028, 1536, 2048, 2052, 2100]


@pytest.mark.parametrize("length", ROW_LENGTHS)
def test_row_kernels_every_dispatch_class(ctx, length):
    """softmax (with a per-row addend), softmax cross-entropy and LayerNorm at row lengths on both sides of
    every lanes-per-row / chunks-per-lane boundary of the row kernels, plus lengths no vector path takes;
    37 rows, so the last wavefront is partly empty."""
    say("row kernels", length)
    rng = np.random.default_rng(length)
    rows = 37
    x = (rng.standard_normal((rows, length)) * 2).astype(np.float32)
    add = rng.standard_normal((rows, 1)).astype(np.float32)
    close(nn.softmax(dev(ctx, x) + dev(ctx, add), 1).eval(ctx).numpy(), O.softmax(O.binary("add", ht(x), ht(add).expand([rows, length])), 1).numpy(),
          REL_MAP, "softmax")
    lab = rng.integers(0, length, (rows, 1)).astype(np.int32)
    loss = nn.softmax_cross_entropy(dev(ctx, x), dev(ctx, lab)).eval(ctx).numpy()
    loss_o = O.softmax_cross_entropy(ht(x), ht(lab.view(np.uint32))).numpy()
    if length == 1:  # one class: the loss is 0 up to the rounding of log(exp(x)); nothing to scale a relative bound by
        assert np.max(np.abs(loss - loss_o)) < 1e-6
    else:
        close(loss, loss_o, REL_MAP, "softmax_cross_entropy")
    if length > 1:
        g = rng.uniform(0.5, 1.5, (length,)).astype(np.float32)
        b = rng.standard_normal((length,)).astype(np.float32)
        close(nn.layer_norm(dev(ctx, x), 1, dev(ctx, g), dev(ctx, b), 1e-5).eval(ctx).numpy(), O.layer_norm(ht(x), 1, ht(g), ht(b), 1e-5).numpy(),
              5e-4, "layer_norm")


# ----------------------------------------------------------------------------- random fills
@pytest.mark.parametrize("shape", [(3, 3), (1000,), (7, 11, 13), (1 << 20,)])
def test_rand_uniform_and_normal(ctx, shape):
    """rand.rs:62-146 for fixed seeds: the uniform fill is integer arithmetic and one multiply (bit-exact);
    the normal fill adds log/sqrt/cos/sin (1e-3 of the largest value)."""
    say("rand", shape)
    sx, sy = 0x9E3779B9, 0x7F4A7C15
    u = V.uniform(list(shape), (sx, sy)).eval(ctx).numpy()
    exact(u, O.rand_uniform(shape, sx, sy).numpy(), "uniform")
    assert u.min() >= 0.0 and u.max() <= 1.0
    z = V.normal(list(shape), (sx, sy)).eval(ctx).numpy()
    zo = O.rand_normal(shape, sx, sy).numpy()
    fin = np.isfinite(zo)  # u1 == 0 gives log(0): the same non-finite values on both sides
    assert np.array_equal(np.isfinite(z), fin)
    assert np.max(np.abs(z[fin] - zo[fin])) < 1e-3 * max(1.0, float(np.abs(zo[fin]).max()))
    # No distribution test: one xorshift step on consecutive seeds is what the reference does, and it is a poor
    # generator (for these seeds the 2^20 "uniform" samples have variance 0.14, the "normal" ones mean 0.65).
    a, b = V.uniform(list(shape)).eval(ctx).numpy(), V.uniform(list(shape)).eval(ctx).numpy()
    assert a.size < 4 or not np.array_equal(a, b)  # unseeded: fresh seeds per evaluation, as the reference
