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


# ---- pins for what the reference holds no vector for ---------------------------------------------------------


def test_xorshift128_known_answers():
    """rand.rs:39-48 worked by hand (32-bit registers; `<<` drops the bits shifted out, `>>` is logical):

        t = x ^ (x << 11);  rndint = y ^ (y >> 19) ^ (t ^ (t >> 8));  return rndint * 2.3283064e-10  [double literal]

    (1, 2):                   t = 0x801,       t ^ (t>>8) = 0x801 ^ 0x8 = 0x809;          y ^ (y>>19) = 2            -> 0x80b = 2059
    (0x80000001, 0xC0000000): x<<11 = 0x800 (bit 31 falls off), t = 0x80000801, t>>8 = 0x00800008 (no sign fill),
                              t ^ (t>>8) = 0x80800809;  y>>19 = 0x1800, y ^ (y>>19) = 0xC0001800               -> 0x40801009
    (0xFFFFFFFF, 0xFFFFFFFF): x<<11 = 0xFFFFF800, t = 0x7FF, t ^ (t>>8) = 0x7FF ^ 0x7 = 0x7F8;  y ^ (y>>19) = 0xFFFFFFFF ^ 0x1FFF
                              = 0xFFFFE000                                                                    -> 0xFFFFE7F8
    The uniform fill evaluates element gid at (seed_x + gid, seed_y + gid) (rand.rs:77-83), so element 0 of a fill
    seeded with the pair is the pair's value.  The last case is a seed on which rounding the double product once
    differs from (float)rndint * 2^-32: rndint = 0x98C4D688, product 0.59675350035.. -> 0x3F18C4D6 (the float-only
    form gives 0x3F18C4D7)."""
    cases = [((1, 2), 2059, 0x3500B000), ((0x80000001, 0xC0000000), 0x40801009, 0x3E810020),
             ((0xFFFFFFFF, 0xFFFFFFFF), 0xFFFFE7F8, 0x3F7FFFE8), ((0x16, 0x98C47536), 0x98C4D688, 0x3F18C4D6)]
    for (sx, sy), rndint, bits in cases:
        u = O.rand_uniform([1], sx, sy).numpy()
        assert u.view(np.uint32)[0] == bits, (hex(sx), hex(sy), hex(int(u.view(np.uint32)[0])))
        # the stored bits are the float nearest to rndint * 2.3283064e-10 (one rounding of the double product)
        assert np.float32(rndint * 2.3283064e-10).view(np.uint32) == bits
    # element gid of a fill uses (seed_x + gid, seed_y + gid), wrapping at 2^32: elements 1 and 2 of a fill seeded
    # (0xFFFFFFFF, 0) are the values of (0, 1) and (1, 2); (0, 1): t = 0, rndint = 1
    u = O.rand_uniform([3], 0xFFFFFFFF, 0).numpy().view(np.uint32)
    assert u[1] == np.float32(1 * 2.3283064e-10).view(np.uint32) and u[2] == 0x3500B000


def test_box_muller_against_float64():
    """rand.rs:120-136: pair p of a normal fill is sqrt(-2 ln u1) * (cos, sin)(2 pi u2) with u1, u2 the uniform values
    of (seed_x + 2p, seed_y) and (seed_x + 2p + 1, seed_y) -- seed_y is NOT advanced, unlike the uniform fill; an odd
    element count keeps the last cosine only.  Uniform values come from the integer step restated here with Python
    integers (pinned above), the transform from float64 `math`."""
    import math

    def u(x, y):
        x &= 0xFFFFFFFF
        t = (x ^ (x << 11)) & 0xFFFFFFFF
        return float(np.float32(((y ^ (y >> 19)) ^ (t ^ (t >> 8))) * 2.3283064e-10))

    sx, sy, n = 0x9E3779B9, 0x7F4A7C15, 9
    z = O.rand_normal([n], sx, sy).numpy()
    for p in range((n + 1) // 2):
        u1, u2 = u(sx + 2 * p, sy), u(sx + 2 * p + 1, sy)
        r = math.sqrt(-2.0 * math.log(u1))
        want = [r * math.cos(2 * math.pi * u2), r * math.sin(2 * math.pi * u2)]
        for j in range(2):
            if 2 * p + j < n:
                assert abs(float(z[2 * p + j]) - want[j]) < 2e-6 * (1.0 + r), (p, j, z[2 * p + j], want[j])
    # closed form: u2 = 0 would give (r, 0); here the invariant z1^2 + z2^2 = -2 ln u1 holds for every full pair
    for p in range(n // 2):
        assert abs(float(z[2 * p]) ** 2 + float(z[2 * p + 1]) ** 2 + 2.0 * math.log(u(sx + 2 * p, sy))) < 1e-5


def test_scatter_against_explicit_loops():
    """core.rs:764-833: for every element of `ind` (coordinates c): y[c with c[axis] := ind[c]] += x[c], y zero-filled
    first; duplicates accumulate.  Nested Python loops on a rank-3 case with duplicate targets along the axis."""
    rng = np.random.default_rng(3)
    x = rng.standard_normal((3, 4, 5)).astype(np.float32)
    for axis, out_ext in ((1, [3, 6, 5]), (0, [4, 4, 5]), (2, [3, 4, 7])):
        ind = rng.integers(0, out_ext[axis], (3, 4, 5)).astype(np.uint32)
        want = np.zeros(out_ext, np.float64)
        for i in range(3):
            for j in range(4):
                for k in range(5):
                    c = [i, j, k]
                    c[axis] = int(ind[i, j, k])
                    want[tuple(c)] += float(x[i, j, k])
        got = O.scatter(T(x), T(ind), axis, out_ext).numpy()
        close(got, want, 1e-5)
        assert np.array_equal(got == 0, want == 0)  # untouched elements are exactly the zero fill
    # an index tensor smaller than x along the axis (the gradient of a [B,1] gather, nn.rs:78-81): only ind's elements move
    ind = rng.integers(0, 10, (3, 1, 5)).astype(np.uint32)
    want = np.zeros((3, 10, 5))
    for i in range(3):
        for k in range(5):
            want[i, ind[i, 0, k], k] += float(x[i, 0, k])
    close(O.scatter(T(x[:, :1, :].copy()), T(ind), 1, [3, 10, 5]).numpy(), want, 1e-6)


@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_gemm_batched_against_explicit_loops(ta, tb):
    """gemm.rs:253-290 + matmul_direct.opencl:170-188: C[b,m,n] = sum_k op(A)[b,m,k] * op(B)[b,k,n] with the stored
    layouts [b,K,M] / [b,N,K] under transposition; nested loops in float64 on a ragged case (a transposed-operand or
    batch-stride mistake moves elements, which a tolerance of 1e-5 on O(1) values does not forgive)."""
    rng = np.random.default_rng(17)
    bt, m, k, n = 3, 5, 7, 4
    a = rng.standard_normal((bt, k, m) if ta else (bt, m, k)).astype(np.float32)
    b = rng.standard_normal((bt, n, k) if tb else (bt, k, n)).astype(np.float32)
    want = np.zeros((bt, m, n))
    for bi in range(bt):
        for i in range(m):
            for j in range(n):
                for kk in range(k):
                    av = a[bi, kk, i] if ta else a[bi, i, kk]
                    bv = b[bi, j, kk] if tb else b[bi, kk, j]
                    want[bi, i, j] += float(av) * float(bv)
    close(O.gemm_batched(T(a), T(b), ta, tb).numpy(), want, 1e-5)
