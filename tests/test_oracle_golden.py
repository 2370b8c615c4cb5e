"""The CPU oracle against every tensor literal the reference's own unit tests hold.

Each test repeats one reference test (file:line in the docstring) through oracle/oracle.py and
compares with the reference's expected literal at the reference's tolerance (max-abs-diff < eps,
tensor.rs:320-328) — integers exactly (tensor.rs:330-341).
"""
import numpy as np
import pytest

from oracle import oracle as O


def close(a, b, eps):
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    assert a.shape == b.shape, (a.shape, b.shape)
    assert np.max(np.abs(a - b)) < eps, np.max(np.abs(a - b))


def T(a):
    return O.HT.from_numpy(a)


def test_nullary_map(golden):
    """map.rs:1383-1391"""
    y = O.scalar(3.0, [3, 3])
    close(y.numpy(), golden("src/ops/map.rs", "test_nullary_map", "y_gt"), 1e-3)


def test_unary_map_sin_and_transposed(golden):
    """map.rs:1394-1440: contiguous and strided-read paths"""
    x = golden("src/ops/map.rs", "test_unary_map", "x")
    y_gt = golden("src/ops/map.rs", "test_unary_map", "y_gt")
    close(O.unary("sin", T(x)).numpy(), y_gt, 1e-3)
    close(O.unary("sin", T(x).transpose(0, 1)).numpy(), y_gt.transpose(1, 0, 2), 1e-3)


def test_binary_map_sub(golden):
    """map.rs:1518-1581"""
    g = lambda n: golden("src/ops/map.rs", "test_binary_map", n)
    close(O.binary("sub", T(g("x1")), T(g("x2"))).numpy(), g("y_gt"), 1e-3)
    close(O.binary("sub", T(g("x1")).tr(), T(g("x2")).tr()).numpy(), g("y_gt").transpose(1, 0, 2), 1e-3)


def test_ternary_map(golden):
    """map.rs:1621-1641: cond(gt(x1, 0), x1, x2)"""
    g = lambda n: golden("src/ops/map.rs", "test_ternary_map", n)
    x1, x2 = T(g("x1")), T(g("x2"))
    close(O.cond(O.binary("gt", x1, 0.0), x1, x2).numpy(), g("y_gt"), 1e-3)


def test_variadic_map(golden):
    """map.rs:1644-1676: ((x1 + x2*3) - x3/2) / x2, un-fused and as one fused launch"""
    g = lambda n: golden("src/ops/map.rs", "test_variadic_map", n)
    x1, x2, x3 = T(g("x1")), T(g("x2")), T(g("x3"))
    y = O.binary("div", O.binary("sub", O.binary("add", x1, O.binary("mul", x2, 3.0)), O.binary("div", x3, 2.0)), x2)
    close(y.numpy(), g("y_gt"), 1e-2)
    E = O.E
    e = E.bin("div", E.bin("sub", E.bin("add", E.inp(0), E.bin("mul", E.inp(1), E.lit(3.0))),
                           E.bin("div", E.inp(2), E.lit(2.0))), E.inp(1))
    yf = O.fused_map(e, [x1, x2, x3], O.FLOAT)
    close(yf.numpy(), g("y_gt"), 1e-2)
    assert np.array_equal(yf.numpy(), y.numpy())


def test_reshape(golden):
    """core.rs:946-991: reshape, and transpose -> reshape (forces the Copy kernel)"""
    g = lambda n: golden("src/ops/core.rs", "test_reshape", n)
    a = T(g("a"))
    b = a.view([4, 2, 3])
    close(b.numpy(), g("b_gt"), 1e-3)
    c = b.transpose(0, 1).view([4, 2, 3])
    close(c.numpy(), g("c_gt"), 1e-3)


def test_expand(golden):
    """core.rs:994-1007"""
    g = lambda n: golden("src/ops/core.rs", "test_expand", n)
    close(T(g("x")).expand([3, 4]).numpy(), g("y_gt"), 1e-3)


def test_permute(golden):
    """core.rs:1010-1062: rank-5 permute [2,3,4,1,0]"""
    g = lambda n: golden("src/ops/core.rs", "test_permute", n)
    y = T(g("x")).permute([2, 3, 4, 1, 0])
    close(y.numpy(), g("y_gt"), 1e-3)
    close(O.unary("copy", y).numpy(), g("y_gt"), 1e-3)  # through the kernel's index translation


def test_slice(golden):
    """core.rs:1076-1105"""
    g = lambda n: golden("src/ops/core.rs", "test_slice", n)
    y = T(g("x")).slice(1, 1, 2)
    close(y.numpy(), g("y_gt"), 1e-3)
    close(O.unary("copy", y).numpy(), g("y_gt"), 1e-3)


def test_unslice(golden):
    """core.rs:1108-1138"""
    g = lambda n: golden("src/ops/core.rs", "test_unslice", n)
    close(O.unslice(T(g("x")), 1, 1, 3).numpy(), g("y_gt"), 1e-3)


def test_gather(golden):
    """core.rs:1141-1190: gather along axis 2"""
    x = golden("src/ops/core.rs", "test_gather", "x")
    t = golden("src/ops/core.rs", "test_gather", "t", np.uint32)
    y_gt = golden("src/ops/core.rs", "test_gather", "y_gt")
    close(O.gather(T(x), T(t), 2).numpy(), y_gt, 1e-3)


def test_concat(golden):
    """core.rs:1196-1232 (the reference only prints the comparison; the literal is still right)"""
    g = lambda n: golden("src/ops/core.rs", "test_concat", n)
    close(O.concat([T(g("x1")), T(g("x2")), T(g("x3"))], 1).numpy(), g("y_gt"), 1e-3)


def test_reduce_mean(golden):
    """reduce.rs:446-486: mean over [0,2,3] of [2,3,2,3,2]"""
    g = lambda n: golden("src/ops/reduce.rs", "test_reduce", n)
    close(O.mean(T(g("x")), [0, 2, 3], False).numpy(), g("y_gt"), 1e-3)


def test_reduce_arg(golden):
    """reduce.rs:501-523: argmax axis 1, exact"""
    x = golden("src/ops/reduce.rs", "test_reduce_arg", "x")
    y_gt = golden("src/ops/reduce.rs", "test_reduce_arg", "y_gt", np.uint32)
    y = O.argmax(T(x), 1, False).numpy()
    assert y.dtype == np.uint32 and np.array_equal(y, y_gt)


def test_gemm(golden):
    """gemm.rs:438-580 (7x13 . 13x5, edge tiles) and :587-709 (7x7 in NN/TN/NT/TT)"""
    g = lambda n: golden("src/ops/gemm.rs", "test_gemm", n)
    close(O.gemm(T(g("a")), T(g("b"))).numpy(), g("c_gt"), 1e-3)
    a, b = T(g("a#2")), T(g("b#2"))
    close(O.gemm(a, b, False, False).numpy(), g("cff_gt"), 1e-3)
    close(O.gemm(a, b, True, False).numpy(), g("ctf_gt"), 1e-3)
    close(O.gemm(a, b, False, True).numpy(), g("cft_gt"), 1e-3)
    close(O.gemm(a, b, True, True).numpy(), g("ctt_gt"), 1e-3)


def test_im2col(golden):
    """conv.rs:545-692: [1,5,4,3], ker (w,h) = [3,2]"""
    g = lambda n: golden("src/ops/conv.rs", "test_im2col", n)
    close(O.im2col(T(g("x")), [3, 2], [1, 1], [0, 0], [1, 1]).numpy(), g("y_gt"), 1e-3)


def test_col2im(golden):
    """conv.rs:699-990: [2,4,2,2,3,3] -> [2,5,4,3], img (w,h) = [4,5], ker (w,h) = [3,2]; plus the adjoint
    identity <im2col(x), c> = <x, col2im(c)> that any col2im must satisfy, with stride, padding and dilation."""
    g = lambda n: golden("src/ops/conv.rs", "test_col2im", n)
    close(O.col2im(T(g("x")), [4, 5], [3, 2], [1, 1], [0, 0], [1, 1]).numpy(), g("y_gt"), 1e-3)
    rng = np.random.default_rng(0)
    for (h, w, c, ker, stride, pad, dil) in [(9, 7, 3, [3, 3], [2, 2], [1, 1], [1, 1]), (11, 10, 2, [3, 2], [2, 1], [0, 1], [2, 2])]:
        x = rng.standard_normal((2, h, w, c)).astype(np.float32)
        xc = O.im2col(T(x), ker, stride, pad, dil).numpy()
        col = rng.standard_normal(xc.shape).astype(np.float32)
        back = O.col2im(T(col), [w, h], ker, stride, pad, dil).numpy()
        lhs, rhs = float((xc.astype(np.float64) * col).sum()), float((x.astype(np.float64) * back).sum())
        assert abs(lhs - rhs) < 1e-3 * max(1.0, abs(lhs))


def test_conv2d(golden):
    """conv.rs:1014-1534: [1,5,5,4] * [3,3,4,8], pad 1"""
    g = lambda n: golden("src/ops/conv.rs", "test_conv2d", n)
    close(O.conv_2d(T(g("x")), T(g("filter")), [1, 1], [1, 1], [1, 1]).numpy(), g("y_gt"), 1e-3)


def test_relu(golden):
    """nn.rs:111-130"""
    g = lambda n: golden("src/ops/nn.rs", "test_relu", n)
    close(O.relu(T(g("x"))).numpy(), g("y_gt"), 1e-3)


def test_softmax(golden):
    """nn.rs:133-154: includes all-negative rows, where the zero-initialised max is harmless"""
    g = lambda n: golden("src/ops/nn.rs", "test_softmax", n)
    close(O.softmax(T(g("x")), 1).numpy(), g("y_gt"), 1e-3)


def test_softmax_cross_entropy(golden):
    """nn.rs:157-207"""
    x = golden("src/ops/nn.rs", "test_softmax_cross_entropy", "x")
    label = golden("src/ops/nn.rs", "test_softmax_cross_entropy", "label", np.uint32)
    loss_gt = golden("src/ops/nn.rs", "test_softmax_cross_entropy", "loss_gt")
    gx_gt = golden("src/ops/nn.rs", "test_softmax_cross_entropy", "gx_gt")
    close(O.softmax_cross_entropy(T(x), T(label)).numpy(), loss_gt, 1e-3)
    # the reference also stores d(loss)/dx = softmax - onehot: an independent check of the forward
    p = O.softmax(T(x), 1).numpy()
    onehot = np.zeros_like(p)
    onehot[np.arange(5), label[:, 0]] = 1
    scale = np.abs(gx_gt).max() / np.abs(p - onehot).max()
    close((p - onehot) * scale, gx_gt, 2e-3)


def test_max_pool_2d(golden):
    """nn.rs:224-348: k3 s1 on [2,5,5,3], tol 1e-2"""
    g = lambda n: golden("src/ops/nn.rs", "test_max_pool_2d", n)
    close(O.max_pool_2d(T(g("x")), 3, 1, 0, 1).numpy(), g("y_gt"), 1e-2)


def test_embedding(golden):
    """layers.rs:619-634: embedding(idx.view([4,1])) == weight.slice(0,0,4)"""
    rng = np.random.default_rng(0)
    w = rng.standard_normal((10, 24)).astype(np.float32)
    idx = golden("src/layers.rs", "test_embedding", "idx", np.int32)
    y = O.embedding(T(w), T(idx).view([4, 1]))
    assert np.array_equal(y.numpy().reshape(4, 24), w[:4])
