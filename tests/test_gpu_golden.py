"""The HIP path (through the C ABI, via the Var front-end) against the reference's own test vectors.

Each test repeats one unit test of the reference (file:line in the docstring), with the reference's
comparison (max-abs-diff < eps, tensor.rs:320-328; integers exactly).  Run on the GPU box: -m gpu.
"""
import numpy as np
import pytest

import sage_amd as S
from sage_amd import nn
from sage_amd import var as V
from sage_amd.layers import Embedding
from sage_amd.shape import Shape

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = S.Context()
    yield c
    c.close()


def dev(ctx, a):
    return S.Var.new(S.Tensor.from_numpy(ctx, a))


def all_close(t, gt, eps):
    a = t.numpy()
    assert list(a.shape) == list(np.shape(gt)), (a.shape, np.shape(gt))
    d = float(np.max(np.abs(a.astype(np.float64) - np.asarray(gt, dtype=np.float64))))
    assert d < eps, d


@pytest.fixture(params=[True, False], ids=["fused", "unfused"])
def fusion(request):
    V.set_fusion(request.param)
    yield request.param
    V.set_fusion(True)


def test_nullary_map(ctx, golden, fusion):
    """map.rs:1383-1391"""
    all_close(V.scalar(3.0, [3, 3]).eval(ctx), golden("src/ops/map.rs", "test_nullary_map", "y_gt"), 1e-3)


def test_unary_map(ctx, golden, fusion):
    """map.rs:1394-1440"""
    x = dev(ctx, golden("src/ops/map.rs", "test_unary_map", "x"))
    y_gt = golden("src/ops/map.rs", "test_unary_map", "y_gt")
    all_close(V.sin(x).eval(ctx), y_gt, 1e-3)
    all_close(V.sin(x.transpose(0, 1)).eval(ctx), y_gt.transpose(1, 0, 2), 1e-3)


def test_binary_map(ctx, golden, fusion):
    """map.rs:1518-1581"""
    g = lambda n: golden("src/ops/map.rs", "test_binary_map", n)
    x1, x2 = dev(ctx, g("x1")), dev(ctx, g("x2"))
    all_close(V.sub(x1, x2).eval(ctx), g("y_gt"), 1e-3)
    all_close(V.sub(V.tr(x1), V.tr(x2)).eval(ctx), g("y_gt").transpose(1, 0, 2), 1e-3)


def test_ternary_map(ctx, golden, fusion):
    """map.rs:1621-1641"""
    g = lambda n: golden("src/ops/map.rs", "test_ternary_map", n)
    x1, x2 = dev(ctx, g("x1")), dev(ctx, g("x2"))
    all_close(V.cond(V.gt(x1, 0.0), x1, x2).eval(ctx), g("y_gt"), 1e-3)


def test_variadic_map(ctx, golden, fusion):
    """map.rs:1644-1676"""
    g = lambda n: golden("src/ops/map.rs", "test_variadic_map", n)
    x1, x2, x3 = dev(ctx, g("x1")), dev(ctx, g("x2")), dev(ctx, g("x3"))
    n0 = ctx.launches
    y = (((x1 + x2 * 3.0) - x3 / 2.0) / x2).eval(ctx)
    all_close(y, g("y_gt"), 1e-2)
    if fusion:
        assert ctx.launches - n0 == 1  # one `variadic` kernel (ops.rs:104-142)


def test_reshape(ctx, golden, fusion):
    """core.rs:946-991"""
    g = lambda n: golden("src/ops/core.rs", "test_reshape", n)
    a = dev(ctx, g("a"))
    b = a.reshape(Shape([4, 2, 3]))
    c = b.transpose(0, 1).reshape(Shape([4, 2, 3]))
    all_close(b.eval(ctx), g("b_gt"), 1e-3)
    all_close(c.eval(ctx), g("c_gt"), 1e-3)


def test_expand(ctx, golden):
    """core.rs:994-1007"""
    g = lambda n: golden("src/ops/core.rs", "test_expand", n)
    all_close(V.expand(dev(ctx, g("x")), [3, 4]).eval(ctx), g("y_gt"), 1e-3)


def test_permute(ctx, golden):
    """core.rs:1010-1062"""
    g = lambda n: golden("src/ops/core.rs", "test_permute", n)
    y = V.permute(dev(ctx, g("x")), [2, 3, 4, 1, 0])
    all_close(y.eval(ctx), g("y_gt"), 1e-3)
    all_close(y.copy().eval(ctx), g("y_gt"), 1e-3)


def test_slice(ctx, golden):
    """core.rs:1076-1105"""
    g = lambda n: golden("src/ops/core.rs", "test_slice", n)
    y = V.slice_(dev(ctx, g("x")), 1, 1, 2)
    all_close(y.eval(ctx), g("y_gt"), 1e-3)
    all_close(y.copy().eval(ctx), g("y_gt"), 1e-3)


def test_unslice(ctx, golden):
    """core.rs:1108-1138"""
    g = lambda n: golden("src/ops/core.rs", "test_unslice", n)
    all_close(V.unslice(dev(ctx, g("x")), 1, 1, 3).eval(ctx), g("y_gt"), 1e-3)


def test_gather(ctx, golden):
    """core.rs:1141-1190"""
    x = dev(ctx, golden("src/ops/core.rs", "test_gather", "x"))
    t = dev(ctx, golden("src/ops/core.rs", "test_gather", "t", np.uint32))
    all_close(V.gather(x, t, 2).eval(ctx), golden("src/ops/core.rs", "test_gather", "y_gt"), 1e-3)


def test_concat(ctx, golden):
    """core.rs:1196-1232"""
    g = lambda n: golden("src/ops/core.rs", "test_concat", n)
    all_close(V.concat([dev(ctx, g("x1")), dev(ctx, g("x2")), dev(ctx, g("x3"))], 1).eval(ctx), g("y_gt"), 1e-3)


def test_reduce(ctx, golden, fusion):
    """reduce.rs:446-486"""
    g = lambda n: golden("src/ops/reduce.rs", "test_reduce", n)
    all_close(V.mean(dev(ctx, g("x")), [0, 2, 3], False).eval(ctx), g("y_gt"), 1e-3)


def test_reduce_arg(ctx, golden):
    """reduce.rs:501-523"""
    x = dev(ctx, golden("src/ops/reduce.rs", "test_reduce_arg", "x"))
    y_gt = golden("src/ops/reduce.rs", "test_reduce_arg", "y_gt", np.uint32)
    y = V.argmax(x, 1, False).eval(ctx).numpy()
    assert y.dtype == np.uint32 and np.array_equal(y, y_gt)


def test_gemm(ctx, golden):
    """gemm.rs:438-709"""
    g = lambda n: golden("src/ops/gemm.rs", "test_gemm", n)
    all_close(V.gemm(dev(ctx, g("a")), dev(ctx, g("b")), False, False).eval(ctx), g("c_gt"), 1e-3)
    a, b = dev(ctx, g("a#2")), dev(ctx, g("b#2"))
    all_close(V.gemm(a, b, False, False).eval(ctx), g("cff_gt"), 1e-3)
    all_close(V.gemm(a, b, True, False).eval(ctx), g("ctf_gt"), 1e-3)
    all_close(V.gemm(a, b, False, True).eval(ctx), g("cft_gt"), 1e-3)
    all_close(V.gemm(a, b, True, True).eval(ctx), g("ctt_gt"), 1e-3)


def test_im2col(ctx, golden):
    """conv.rs:545-692"""
    g = lambda n: golden("src/ops/conv.rs", "test_im2col", n)
    all_close(V.im2col(dev(ctx, g("x")), [3, 2], [1, 1], [0, 0], [1, 1]).eval(ctx), g("y_gt"), 1e-3)


def test_conv2d(ctx, golden, fusion):
    """conv.rs:1014-1534"""
    g = lambda n: golden("src/ops/conv.rs", "test_conv2d", n)
    y = V.conv_2d(dev(ctx, g("x")), dev(ctx, g("filter")), [1, 1], [1, 1], [1, 1])
    all_close(y.eval(ctx), g("y_gt"), 1e-3)


def test_relu(ctx, golden, fusion):
    """nn.rs:111-130"""
    g = lambda n: golden("src/ops/nn.rs", "test_relu", n)
    all_close(nn.relu(dev(ctx, g("x"))).eval(ctx), g("y_gt"), 1e-3)


def test_softmax(ctx, golden, fusion):
    """nn.rs:133-154"""
    g = lambda n: golden("src/ops/nn.rs", "test_softmax", n)
    all_close(nn.softmax(dev(ctx, g("x")), 1).eval(ctx), g("y_gt"), 1e-3)


def test_softmax_cross_entropy(ctx, golden, fusion):
    """nn.rs:157-207"""
    x = dev(ctx, golden("src/ops/nn.rs", "test_softmax_cross_entropy", "x"))
    label = dev(ctx, golden("src/ops/nn.rs", "test_softmax_cross_entropy", "label", np.uint32))
    all_close(nn.softmax_cross_entropy(x, label).eval(ctx), golden("src/ops/nn.rs", "test_softmax_cross_entropy", "loss_gt"), 1e-3)


def test_max_pool_2d(ctx, golden):
    """nn.rs:224-348"""
    g = lambda n: golden("src/ops/nn.rs", "test_max_pool_2d", n)
    all_close(V.max_pool_2d(dev(ctx, g("x")), 3, 1, 0, 1).eval(ctx), g("y_gt"), 1e-2)


def test_embedding(ctx, golden):
    """layers.rs:619-634: embedding(idx.view([4,1])) == weight.slice(0,0,4)"""
    rng = np.random.default_rng(0)
    w = rng.standard_normal((10, 24)).astype(np.float32)
    emb = Embedding(10, 24)
    emb.weight.set(S.Tensor.from_numpy(ctx, w))
    idx = dev(ctx, golden("src/layers.rs", "test_embedding", "idx", np.int32))
    y = emb.pass_(idx.view([4, 1])).eval(ctx).numpy()
    y_gt = emb.weight.slice(0, 0, 4).eval(ctx).numpy()
    assert np.array_equal(y.reshape(4, 24), y_gt)
