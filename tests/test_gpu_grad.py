"""Backward path: gradient graphs (sage_amd/grad.py, mirror of var.rs:56-103 and every operator's
`grad`), col2im, and the optimizers, on the GPU.

What pins what: col2im is checked bit for bit against the oracle's restatement and the reference's
own vectors (conv.rs:699-990); the gradient RULES are checked against torch autograd in float64 on the
same expressions (an independent derivation) and against the reference's softmax-CE gradient fixture
(nn.rs:181-197); the optimizer arithmetic against a numpy restatement of optim.rs."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import sage_amd as S
from oracle import oracle as O
from sage_amd import nn, optim
from sage_amd import var as V
from sage_amd.bert import BertConfig, BertLayer
from sage_amd.grad import grad, grad_check, grad_param
from sage_amd.layers import load_params
from sage_amd.resnet import ResNet, ResNetConfig
from tests.test_gpu_models import bert_layer_params, layer_param_list, resnet_arrays, torch_bert_layer
from tests.util import REL_GEMM, REL_MAP, close, exact

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = S.Context()
    yield c
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


def t64(a):
    return torch.tensor(np.asarray(a, np.float64), requires_grad=True)


# ----------------------------------------------------------------------------- col2im
def test_col2im_reference_vector(ctx, golden):
    say("col2im golden")
    x = golden("src/ops/conv.rs", "test_col2im", "x")
    want = golden("src/ops/conv.rs", "test_col2im", "y_gt")
    y = V.col2im(dev(ctx, x), [4, 5], [3, 2], [1, 1], [0, 0], [1, 1]).eval(ctx).numpy()
    assert np.max(np.abs(y - want)) < 1e-3  # the reference's own tolerance (conv.rs:989)
    exact(y, O.col2im(ht(x), [4, 5], [3, 2], [1, 1], [0, 0], [1, 1]).numpy(), "vs oracle")


@pytest.mark.parametrize("n,h,w,c,ker,stride,pad,dil", [
    (2, 9, 7, 3, [3, 3], [1, 1], [1, 1], [1, 1]), (3, 14, 14, 8, [3, 3], [2, 2], [1, 1], [1, 1]),
    (1, 28, 28, 1, [7, 7], [2, 2], [3, 3], [1, 1]), (2, 8, 8, 4, [1, 1], [2, 2], [0, 0], [1, 1]),
    (2, 11, 10, 2, [3, 2], [2, 1], [0, 1], [2, 2]), (1, 7, 7, 64, [3, 3], [1, 1], [1, 1], [1, 1]),
    (2, 12, 9, 8, [5, 3], [3, 2], [2, 1], [1, 1]), (1, 6, 5, 4, [2, 2], [3, 3], [0, 0], [1, 1]),  # stride above the kernel: pixels no tap reads
    # two different dilations: the reference's kernel defines no result (it takes tap indices from the wrong dilation,
    # conv.rs:463-465), the oracle refuses, the product returns the adjoint (checked by the identity below)
    (2, 11, 10, 4, [3, 2], [1, 2], [1, 1], [1, 2]), (1, 9, 12, 3, [2, 3], [2, 1], [2, 0], [3, 1])])
def test_col2im_vs_oracle_and_adjoint(ctx, n, h, w, c, ker, stride, pad, dil):
    say("col2im", n, h, w, c, ker, stride, pad, dil)
    rng = np.random.default_rng(h * 100 + w)
    ow, oh = V.conv_size([w, h], ker, stride, pad, dil)
    col = rng.standard_normal((n, oh, ow, ker[1], ker[0], c)).astype(np.float32)
    y = V.col2im(dev(ctx, col), [w, h], ker, stride, pad, dil).eval(ctx).numpy()
    if dil[0] == dil[1]:
        exact(y, O.col2im(ht(col), [w, h], ker, stride, pad, dil).numpy(), "vs oracle")
    else:
        with pytest.raises(RuntimeError, match="or_col2im"):
            O.col2im(ht(col), [w, h], ker, stride, pad, dil)
        # every pixel is the float64 sum of the entries im2col's index map sends to it (an explicit scatter of indices)
        idx = np.arange(n * h * w * c, dtype=np.float64).reshape(n, h, w, c) + 1.0  # im2col of pixel numbers; 0 marks padding
        src = O.im2col(ht(idx.astype(np.float32)), ker, stride, pad, dil).numpy().astype(np.int64).ravel()
        want = np.zeros(n * h * w * c + 1)
        np.add.at(want, src, col.astype(np.float64).ravel())
        close(y, want[1:].reshape(n, h, w, c), 1e-5, "col2im vs the scatter of im2col's index map")
    # adjoint identity: <im2col(x), col> == <x, col2im(col)>
    x = rng.standard_normal((n, h, w, c)).astype(np.float32)
    xc = V.im2col(dev(ctx, x), ker, stride, pad, dil).eval(ctx).numpy()
    lhs, rhs = float((xc.astype(np.float64) * col).sum()), float((x.astype(np.float64) * y).sum())
    assert abs(lhs - rhs) <= 1e-4 * max(1.0, abs(lhs)), (lhs, rhs)


# ----------------------------------------------------------------------------- operator rules vs torch
def check_grads(ctx, build, build_torch, arrays, rel=REL_MAP, seed_shape=None):
    """build(*Vars) -> Var y ; build_torch(*tensors) -> tensor y.  Compares d(sum(w*y))/d(inputs)."""
    rng = np.random.default_rng(99)
    vs = [dev(ctx, a) for a in arrays]
    y = build(*vs)
    w = rng.standard_normal(y.extents).astype(np.float32)
    gs = grad(y, vs, seed=dev(ctx, w))
    ts = [t64(a) for a in arrays]
    yt = build_torch(*ts)
    assert list(yt.shape) == y.extents, (yt.shape, y.extents)
    (yt * torch.tensor(w.astype(np.float64))).sum().backward()
    for i, (g, t) in enumerate(zip(gs, ts)):
        close(g.eval(ctx).numpy(), t.grad.numpy(), rel, f"gradient of input {i}")


UNARY_T = {
    "abs": torch.abs, "neg": torch.neg, "recip": torch.reciprocal, "log": torch.log, "exp": torch.exp, "sqrt": torch.sqrt,
    "square": torch.square, "erf": torch.erf, "sin": torch.sin, "sinh": torch.sinh, "cos": torch.cos, "cosh": torch.cosh,
    "tan": torch.tan, "tanh": torch.tanh, "asin": torch.asin, "asinh": torch.asinh, "acos": torch.acos, "acosh": torch.acosh,
    "atan": torch.atan, "atanh": torch.atanh, "copy": lambda t: t * 1.0,
}
DOMAIN = {"log": (0.2, 3), "sqrt": (0.2, 3), "recip": (0.5, 2), "acosh": (1.2, 4), "asin": (-0.9, 0.9), "acos": (-0.9, 0.9),
          "atanh": (-0.9, 0.9), "tan": (-1.2, 1.2), "abs": (0.1, 2)}


@pytest.mark.parametrize("name", sorted(UNARY_T))
def test_unary_map_gradients(ctx, name):
    say("grad unary", name)
    lo, hi = DOMAIN.get(name, (-1.5, 1.5))
    x = np.random.default_rng(len(name)).uniform(lo, hi, (5, 7)).astype(np.float32)
    check_grads(ctx, lambda v: V.unary_map(v, name), UNARY_T[name], [x], rel=5e-4)


def test_unary_map_zero_gradients(ctx):
    say("grad sign/ceil/floor/round")
    x = np.random.default_rng(3).uniform(-2, 2, (4, 4)).astype(np.float32)
    for name in ("sign", "ceil", "floor", "round"):
        v = dev(ctx, x)
        g = grad(V.unary_map(v, name), [v])[0].eval(ctx).numpy()
        exact(g, np.zeros_like(x), name)


@pytest.mark.parametrize("name,fn", [("add", torch.add), ("sub", torch.sub), ("mul", torch.mul), ("div", torch.div),
                                     ("pow", torch.pow), ("min", torch.minimum), ("max", torch.maximum)])
def test_binary_map_gradients_with_broadcast(ctx, name, fn):
    say("grad binary", name)
    rng = np.random.default_rng(7)
    a = rng.uniform(0.5, 2.0, (3, 4, 5)).astype(np.float32)
    b = rng.uniform(0.5, 2.0, (4, 1)).astype(np.float32)  # broadcast: exercises Expand::grad (core.rs:292-313)
    check_grads(ctx, lambda x, y: V.binary_map(x, y, name), fn, [a, b], rel=5e-4)


def test_cond_gradient_is_the_references(ctx):
    """map.rs:1094-1099 hands cond(c, gy, 0) to the CONDITION input and cond(c, 0, gy) to the first branch."""
    say("grad cond")
    rng = np.random.default_rng(8)
    x1, x2 = rng.standard_normal((4, 6)).astype(np.float32), rng.standard_normal((4, 6)).astype(np.float32)
    w = rng.standard_normal((4, 6)).astype(np.float32)
    v1, v2 = dev(ctx, x1), dev(ctx, x2)
    c = V.gt(v1, 0.0)
    y = V.cond(c, v1, v2)
    g1 = grad(y, [v1], seed=dev(ctx, w))[0].eval(ctx).numpy()
    exact(g1, np.where(x1 > 0, 0.0, w).astype(np.float32), "first branch gets cond(c, 0, gy)")
    with pytest.raises(KeyError):
        grad(y, [v2])


@pytest.mark.parametrize("op,axes", [("sum", [1]), ("sum", [0, 2]), ("prod", [2]), ("max", [1]), ("min", [0])])
@pytest.mark.parametrize("keep", [False, True])
def test_reduce_gradients(ctx, op, axes, keep):
    say("grad reduce", op, axes, keep)
    x = np.random.default_rng(len(axes)).uniform(0.5, 2.0, (3, 4, 5)).astype(np.float32)
    tfn = {"sum": lambda t: t.sum(axes, keepdim=keep), "prod": lambda t: t.prod(axes[0], keepdim=keep),
           "max": lambda t: t.amax(axes, keepdim=keep), "min": lambda t: t.amin(axes, keepdim=keep)}[op]
    # init="identity": with the reference's zero-initialised accumulator (reduce.rs:282) a product is always 0 and
    # a minimum of positive data is 0, and so are their gradients; the rule itself is what is compared here
    check_grads(ctx, lambda v: V.reduce(v, axes, keep, op, init="identity"), tfn, [x], rel=5e-4)


def test_mean_var_gradients(ctx):
    say("grad mean/var")
    x = np.random.default_rng(5).standard_normal((6, 10)).astype(np.float32)
    check_grads(ctx, lambda v: v.mean([1], True), lambda t: t.mean(1, keepdim=True), [x])
    check_grads(ctx, lambda v: v.var([1], False), lambda t: t.var(1, unbiased=False), [x], rel=5e-4)


def test_layout_and_index_gradients(ctx):
    say("grad layout/index ops")
    rng = np.random.default_rng(11)
    x = rng.standard_normal((4, 5, 6)).astype(np.float32)
    check_grads(ctx, lambda v: v.transpose(0, 2), lambda t: t.transpose(0, 2), [x])
    check_grads(ctx, lambda v: v.transpose(1, 2).view([4, 30]), lambda t: t.transpose(1, 2).reshape(4, 30), [x])
    check_grads(ctx, lambda v: v.slice(1, 1, 4), lambda t: t[:, 1:4], [x])
    check_grads(ctx, lambda v: v.unslice(2, 3, 12), lambda t: F.pad(t, (3, 3)), [x])
    check_grads(ctx, lambda v: v.unsqueeze(1).squeeze(1).expand([2, 4, 5, 6]), lambda t: t.expand(2, 4, 5, 6), [x])
    y = rng.standard_normal((4, 2, 6)).astype(np.float32)
    check_grads(ctx, lambda a, b: V.concat([a, b, a], 1), lambda a, b: torch.cat([a, b, a], 1), [x, y])
    ind = rng.integers(0, 5, (4, 3, 6)).astype(np.int32)
    ti = torch.tensor(ind.astype(np.int64))
    check_grads(ctx, lambda v: v.gather(dev(ctx, ind), 1), lambda t: torch.gather(t, 1, ti), [x])
    perm = np.stack([rng.permutation(5) for _ in range(4 * 6)]).reshape(4, 6, 5).transpose(0, 2, 1).astype(np.int32)
    tp = torch.tensor(perm.astype(np.int64))
    check_grads(ctx, lambda v: v.scatter(dev(ctx, perm), 1, [4, 5, 6]), lambda t: torch.zeros(4, 5, 6, dtype=torch.float64).scatter_add(1, tp, t), [x])


@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_gemm_gradients(ctx, ta, tb):
    say("grad gemm", ta, tb)
    rng = np.random.default_rng(13)
    m, k, n = 9, 14, 6
    a = rng.standard_normal((k, m) if ta else (m, k)).astype(np.float32)
    b = rng.standard_normal((n, k) if tb else (k, n)).astype(np.float32)
    tf = lambda x, y: (x.T if ta else x) @ (y.T if tb else y)
    check_grads(ctx, lambda x, y: V.gemm(x, y, ta, tb), tf, [a, b], rel=REL_GEMM)
    a3, b3 = np.stack([a, a * 0.5, -a]), np.stack([b, b + 1, b * 2])
    tf3 = lambda x, y: (x.transpose(1, 2) if ta else x) @ (y.transpose(1, 2) if tb else y)
    check_grads(ctx, lambda x, y: V.gemm_batched(x, y, ta, tb), tf3, [a3, b3], rel=REL_GEMM)


def test_dense_and_attention_chain_gradients(ctx):
    """matmul + bias (layers.rs:243-247) and the attention chain of bert.rs:262-271 with the fused nodes
    (matmul_nd, softmax, sg_attention in the forward pass): gradients go through the reference's composition."""
    say("grad dense / attention")
    rng = np.random.default_rng(17)
    x, w, b = rng.standard_normal((2, 5, 8)).astype(np.float32), rng.standard_normal((8, 6)).astype(np.float32), rng.standard_normal(6).astype(np.float32)
    check_grads(ctx, lambda x_, w_, b_: x_.matmul(w_) + b_, lambda x_, w_, b_: x_ @ w_ + b_, [x, w, b], rel=REL_GEMM)
    n, h, l, d = 2, 2, 16, 32
    q, k, v = (rng.standard_normal((n, l, h * d)).astype(np.float32) for _ in range(3))

    def heads(f):
        return f.view([n, l, h, d]).transpose(2, 1)

    def build(q_, k_, v_):
        att = heads(q_).matmul_batched(heads(k_).transpose(-1, -2)) * 0.25
        return nn.softmax(att, 3).matmul_batched(heads(v_)).transpose(2, 1).view([n, l, h * d])

    def build_t(q_, k_, v_):
        hs = lambda f: f.reshape(n, l, h, d).transpose(1, 2)
        att = torch.softmax(hs(q_) @ hs(k_).transpose(-1, -2) * 0.25, -1)
        return (att @ hs(v_)).transpose(1, 2).reshape(n, l, h * d)

    check_grads(ctx, build, build_t, [q, k, v], rel=REL_GEMM)


def test_layer_norm_and_softmax_ce_gradients(ctx, golden):
    say("grad layer_norm / softmax_ce")
    rng = np.random.default_rng(19)
    x = rng.standard_normal((6, 24)).astype(np.float32)
    g, b = rng.uniform(0.5, 1.5, 24).astype(np.float32), rng.standard_normal(24).astype(np.float32)
    check_grads(ctx, lambda x_, g_, b_: nn.layer_norm(x_, 1, g_, b_, 1e-5), lambda x_, g_, b_: F.layer_norm(x_, (24,), g_, b_, 1e-5),
                [x, g, b], rel=5e-4)
    lab = rng.integers(0, 24, (6, 1)).astype(np.int32)
    tl = torch.tensor(lab[:, 0].astype(np.int64))
    check_grads(ctx, lambda x_: nn.softmax_cross_entropy(x_, dev(ctx, lab)), lambda x_: F.cross_entropy(x_, tl, reduction="none"), [x], rel=5e-4)
    # the reference's fixture: d mean(loss) / d x  (nn.rs:157-207)
    xs = golden("src/ops/nn.rs", "test_softmax_cross_entropy", "x")
    ts = golden("src/ops/nn.rs", "test_softmax_cross_entropy", "label", np.int32).reshape(-1, 1)
    gx = golden("src/ops/nn.rs", "test_softmax_cross_entropy", "gx_gt")
    xv = dev(ctx, xs)
    loss = nn.softmax_cross_entropy(xv, dev(ctx, ts)).mean(0, False)
    assert np.max(np.abs(grad(loss, [xv])[0].eval(ctx).numpy() - gx)) < 1e-3


@pytest.mark.parametrize("stride,pad", [(1, 1), (2, 1), (2, 0)])
def test_conv_and_pool_gradients(ctx, stride, pad):
    say("grad conv2d / pools", stride, pad)
    rng = np.random.default_rng(23 + stride)
    x = rng.standard_normal((2, 9, 8, 3)).astype(np.float32)
    w = rng.standard_normal((3, 3, 3, 5)).astype(np.float32) * 0.3
    tconv = lambda x_, w_: F.conv2d(x_.permute(0, 3, 1, 2), w_.permute(3, 2, 0, 1), stride=stride, padding=pad).permute(0, 2, 3, 1)
    check_grads(ctx, lambda x_, w_: V.conv_2d(x_, w_, stride, pad, 1), tconv, [x, w], rel=REL_GEMM)
    xp = np.abs(x) + 0.1  # positive: the reference's zero-initialised max accumulator is not in play
    tmax = lambda x_: F.max_pool2d(x_.permute(0, 3, 1, 2), 3, stride, pad).permute(0, 2, 3, 1)
    check_grads(ctx, lambda x_: V.max_pool_2d(x_, 3, stride, pad, 1), tmax, [xp])
    tavg = lambda x_: F.avg_pool2d(x_.permute(0, 3, 1, 2), 3, stride, pad, count_include_pad=True).permute(0, 2, 3, 1)
    check_grads(ctx, lambda x_: V.avg_pool_2d(x_, 3, stride, pad, 1), tavg, [x])


def test_grad_check_finite_differences(ctx):
    """The reference's own way of testing a gradient (var.rs:107-150), on col2im (conv.rs:990) and a map chain."""
    say("grad_check")
    rng = np.random.default_rng(29)
    col = dev(ctx, rng.standard_normal((1, 3, 2, 2, 3, 2)).astype(np.float32))
    assert grad_check(V.col2im(col, [4, 4], [3, 2], [1, 1], [0, 0], [1, 1]), col, 0.01, ctx, eps=1e-2)
    x = dev(ctx, rng.uniform(0.5, 1.5, (3, 4)).astype(np.float32))
    assert grad_check((x.square() * 3.0 + x.log()).sum([1], False), x, 0.05, ctx, eps=1e-2)


# ----------------------------------------------------------------------------- whole models
def torch_resnet18(x, p):
    def conv(t, w, b, stride, pad):
        return F.conv2d(t.permute(0, 3, 1, 2), w.permute(3, 2, 0, 1), b, stride=stride, padding=pad).permute(0, 2, 3, 1)
    y = torch.relu(conv(x, p["w0"], p["b0"], 2, 3))
    y = F.max_pool2d(y.permute(0, 3, 1, 2), 3, 2, 1).permute(0, 2, 3, 1)
    for blk in p["blocks"]:
        z = torch.relu(conv(y, blk["w1"], blk["b1"], blk["stride"], 1))
        z = conv(z, blk["w2"], blk["b2"], 1, 1)
        sc = conv(y, blk["wd"], blk["bd"], blk["stride"], 0) if "wd" in blk else y
        y = torch.relu(z + sc)
    y = y.mean((1, 2))
    return y @ p["wfc"] + p["bfc"]


def test_resnet18_training_step_vs_torch_and_adam(ctx):
    """examples/train.rs: loss = mean softmax-CE of ResNet-18 logits, grad_param, Adam.  Loss and all 42
    parameter gradients against torch autograd (float64); three Adam updates against optim.rs restated in numpy."""
    say("resnet18 train step")
    rng = np.random.default_rng(31)
    arrays, po = resnet_arrays(rng, 1, 10)
    model = ResNet(ResNetConfig.d18(1, 10))
    load_params(ctx, model, arrays)
    n = 8
    x = rng.uniform(0, 1, (n, 28, 28, 1)).astype(np.float32)
    lab = rng.integers(0, 10, (n, 1)).astype(np.int32)
    xv, lv = dev(ctx, x), dev(ctx, lab)
    logits = model.pass_(xv)
    loss = nn.softmax_cross_entropy(logits, lv).mean(0, False)
    grads = grad_param(loss, model)
    prog = S.Program(ctx, list(grads.values()) + [loss]).bind()

    tp = {"w0": t64(po["w0"]), "b0": t64(po["b0"]), "wfc": t64(po["wfc"]), "bfc": t64(po["bfc"]), "blocks": []}
    order = [tp["w0"], tp["b0"]]
    for b in po["blocks"]:
        tb = {k: (t64(v) if isinstance(v, np.ndarray) else v) for k, v in b.items()}
        tp["blocks"].append(tb)
        order += [tb["w1"], tb["b1"], tb["w2"], tb["b2"]] + ([tb["wd"], tb["bd"]] if "wd" in tb else [])
    order += [tp["wfc"], tp["bfc"]]
    tl = F.cross_entropy(torch_resnet18(torch.tensor(x.astype(np.float64)), tp), torch.tensor(lab[:, 0].astype(np.int64)))
    tl.backward()
    close(prog.outputs[-1].numpy(), np.array([tl.item()]), REL_GEMM, "loss")
    g0 = [o.numpy().copy() for o in prog.outputs[:-1]]
    for i, (g, t) in enumerate(zip(g0, order)):
        close(g, t.grad.numpy(), 2e-3, f"gradient of parameter {i}")

    # Adam, three updates on a fixed batch (optim.rs:133-177): state appears at the first update as zeros
    opt = optim.Adam(1e-3)
    opt.init(ctx)
    params = list(grads.keys())
    w = [p.value.numpy().astype(np.float64) for p in params]
    m = [None] * len(w)
    v = [None] * len(w)
    t = 1.0
    for step in range(3):
        prog.run()
        gs = [o.numpy().astype(np.float64) for o in prog.outputs[:-1]]
        opt.update(grads, ctx)
        for i, g in enumerate(gs):
            m[i] = np.zeros_like(g) if m[i] is None else m[i] * B1 + g * OMB1
            v[i] = np.zeros_like(g) if v[i] is None else v[i] * B2 + g ** 2 * OMB2
            w[i] = w[i] - (m[i] / (1.0 - B1 ** t)) * 1e-3 / (np.sqrt(v[i] / (1.0 - B2 ** t)) + 1e-8)
        t += 1.0
        for i, p in enumerate(params):
            close(p.value.numpy(), w[i], 2e-3, f"step {step} parameter {i}")
        if step == 0:
            exact(params[0].value.numpy(), arrays[0], "the first Adam update leaves the weights as they were")
    assert not np.array_equal(params[0].value.numpy(), arrays[0])

    # the same update as a replayable Program: building it is update 4, every run() one more; also as a HIP graph
    def numpy_step(gs):
        nonlocal t
        for i, g in enumerate(gs):
            m[i] = m[i] * B1 + g * OMB1
            v[i] = v[i] * B2 + g ** 2 * OMB2
            w[i] = w[i] - (m[i] / (1.0 - B1 ** t)) * 1e-3 / (np.sqrt(v[i] / (1.0 - B2 ** t)) + 1e-8)
        t += 1.0

    prog.run()
    numpy_step([o.numpy().astype(np.float64) for o in prog.outputs[:-1]])
    upd = opt.compile(grads, ctx)
    for use_graph in (False, True):
        if use_graph:
            upd.capture()
        for _ in range(2):
            prog.run()
            numpy_step([o.numpy().astype(np.float64) for o in prog.outputs[:-1]])
            upd.run()
    upd.release_graph()
    for i, p in enumerate(params):
        close(p.value.numpy(), w[i], 3e-3, f"compiled updates, parameter {i}")
    close(opt.t.numpy(), np.array([t]), 1e-6, "step counter")


def test_bert_layer_gradients_vs_torch(ctx):
    say("bert layer grads")
    rng = np.random.default_rng(37)
    n, l, e, heads, hdim = 2, 16, 64, 2, 128
    p = bert_layer_params(rng, e, hdim, per_feature=True)
    layer = BertLayer(BertConfig(e, 100, 512, hdim, 1, heads, 1e-12, 0.1, 2), reference_exact=False)
    load_params(ctx, layer, layer_param_list(p))
    x = rng.standard_normal((n, l, e)).astype(np.float32)
    mask = np.ones((n, l), np.float32)
    mask[1, 12:] = 0.0
    w = rng.standard_normal((n, l, e)).astype(np.float32)
    xv = dev(ctx, x)
    y = layer.pass_(xv, dev(ctx, mask))
    params = layer.params()
    gs = grad(y, params + [xv], seed=dev(ctx, w))
    tp = {k: t64(v) for k, v in p.items()}
    tx = t64(x)
    yt = torch_bert_layer(tx, torch.tensor(mask.astype(np.float64)), tp, heads, "gelu", 1e-12)
    (yt * torch.tensor(w.astype(np.float64))).sum().backward()
    close(y.eval(ctx).numpy(), yt.detach().numpy(), REL_GEMM, "forward")
    keys = ["wk", "bk", "wq", "bq", "wv", "bv", "wo", "bo", "ln1_g", "ln1_b", "w1", "b1", "w2", "b2", "ln2_g", "ln2_b"]
    for k, g in zip(keys, gs[:-1]):
        if k == "bk":  # a key bias shifts every score of a row alike: its gradient is zero up to rounding
            assert np.max(np.abs(g.eval(ctx).numpy())) < 1e-5 and np.max(np.abs(tp[k].grad.numpy())) < 1e-12
            continue
        close(g.eval(ctx).numpy(), tp[k].grad.numpy(), 2e-3, "gradient of " + k)
    close(gs[-1].eval(ctx).numpy(), tx.grad.numpy(), 2e-3, "gradient of the input")


def test_sgd_plain_and_reference_momentum_bug(ctx):
    say("sgd")
    rng = np.random.default_rng(41)
    w0 = rng.standard_normal((4, 3)).astype(np.float32)
    p = dev(ctx, w0)
    loss = (p.square() * 0.5).sum([0, 1], False)
    grads = {p: grad(loss, [p])[0]}
    optim.Sgd(0.1).update(grads, ctx)
    close(p.value.numpy(), w0 - 0.1 * w0, 1e-6, "w - lr * w")
    with pytest.raises(KeyError):  # optim.rs:67-69: the reference indexes a missing momentum entry
        optim.Sgd(0.1, momentum=0.9).update({p: grad(loss, [p])[0]}, ctx)


def test_fused_sibling_dense_follows_parameter_updates(ctx):
    """q/k/v projections sharing an input run as one GEMM on concatenated weights.  The concatenation is derived
    data: after the parameters are rewritten in place (an optimizer step, a host write) a replayed Program and
    a fresh evaluation must both see the new weights."""
    say("wide weights after updates")
    rng = np.random.default_rng(43)
    n, l, e, heads, hdim = 2, 16, 64, 2, 128
    p = bert_layer_params(rng, e, hdim, per_feature=True)
    layer = BertLayer(BertConfig(e, 100, 512, hdim, 1, heads, 1e-12, 0.1, 2), reference_exact=False)
    load_params(ctx, layer, layer_param_list(p))
    x = rng.standard_normal((n, l, e)).astype(np.float32)
    mask = np.ones((n, l), np.float32)
    xv, mv = dev(ctx, x), dev(ctx, mask)
    y = layer.pass_(xv, mv)
    prog = S.Program(ctx, [y])
    close(prog.run()[0].numpy(), torch_bert_layer(x, mask, p, heads, "gelu", 1e-12), REL_GEMM, "before")
    loss = y.square().sum([0, 1, 2], False)
    grads = dict(zip(layer.params(), grad(loss, layer.params())))
    optim.Sgd(0.05).update(grads, ctx)
    keys = ["wk", "bk", "wq", "bq", "wv", "bv", "wo", "bo", "ln1_g", "ln1_b", "w1", "b1", "w2", "b2", "ln2_g", "ln2_b"]
    p2 = {k: v.value.numpy() for k, v in zip(keys, layer.params())}
    assert not np.array_equal(p2["wq"], p["wq"])
    want = torch_bert_layer(x, mask, p2, heads, "gelu", 1e-12)
    close(prog.run()[0].numpy(), want, REL_GEMM, "replayed Program after the update")
    close(layer.pass_(xv, mv).eval(ctx).numpy(), want, REL_GEMM, "fresh evaluation after the update")
    prog.capture()
    layer.params()[2].value.copy_from_numpy(p["wq"])  # host write into the query weights
    p2["wq"] = p["wq"]
    close(prog.run()[0].numpy(), torch_bert_layer(x, mask, p2, heads, "gelu", 1e-12), REL_GEMM, "graph replay after a host write")
    prog.release_graph()


# Adam's hyper-parameters are f32 fields in the reference and `1.0 - self.beta` is an f32 subtraction (optim.rs:152, 160):
# the float64 restatements below use those f32 values (1 - 0.999f = 0.0009999871, which is 1.3e-5 away from 0.001).
B1, B2 = float(np.float32(0.9)), float(np.float32(0.999))
OMB1, OMB2 = float(np.float32(1.0) - np.float32(0.9)), float(np.float32(1.0) - np.float32(0.999))


ADAM_SHAPES = [(1,), (3,), (5, 7), (64,), (33, 17), (128, 96), (4100,), (2, 3, 4, 5), (1024,), (1025,), (7, 7, 1, 64)] + \
    [(16 + i,) for i in range(24)] + [(3, 3, 64, 64)]


@pytest.mark.parametrize("weight_decay", [0.0, 0.01])
def test_adam_fused_update_is_the_operator_chain(ctx, weight_decay):
    """sg_adam_update (all parameters in one or two launches, in place) against Adam::update replayed as the
    reference's map operators (optim.rs:129-177): bit-identical values, moments and step counter over several
    steps with changing gradients, eager and as a HIP graph; 36 tensors (two launches), sizes around the
    4-element and 1024-element boundaries; and against the expressions in float64."""
    say("adam fused", weight_decay)
    rng = np.random.default_rng(53)
    w0 = [rng.standard_normal(s).astype(np.float32) for s in ADAM_SHAPES]
    g_steps = [[(rng.standard_normal(s) * 0.1).astype(np.float32) for s in ADAM_SHAPES] for _ in range(6)]

    def make():
        params = [dev(ctx, w) for w in w0]
        gvars = [dev(ctx, g) for g in g_steps[0]]
        return params, gvars, dict(zip(params, gvars)), optim.Adam(1e-2, weight_decay=weight_decay)

    def feed(gvars, gs):
        for gv, g in zip(gvars, gs):
            gv.value.copy_from_numpy(g)

    pa, ga, grads_a, opt_a = make()
    pb, gb, grads_b, opt_b = make()
    w = [x.astype(np.float64) for x in w0]
    m = [np.zeros_like(x) for x in w]
    v = [np.zeros_like(x) for x in w]
    t = 1.0

    def numpy_step(gs, first=False):
        nonlocal t
        for i, g in enumerate(gs):
            g = g.astype(np.float64) + w[i] * weight_decay if weight_decay else g.astype(np.float64)
            if not first:
                m[i] = m[i] * B1 + g * OMB1
                v[i] = v[i] * B2 + g ** 2 * OMB2
            w[i] = w[i] - (m[i] / (1.0 - B1 ** t)) * 1e-2 / (np.sqrt(v[i] / (1.0 - B2 ** t)) + 1e-8)
        t += 1.0

    for step in range(2):  # the first update stores zero moments (optim.rs:149-163), the second accumulates
        for gv, o in ((ga, opt_a), (gb, opt_b)):
            feed(gv, g_steps[step])
        opt_a.update(grads_a, ctx)
        opt_b.update(grads_b, ctx)
        numpy_step(g_steps[step], first=step == 0)
    feed(ga, g_steps[2]); feed(gb, g_steps[2])
    n0 = ctx.launches
    prog_a = opt_a.compile(grads_a, ctx)                 # building performs update 3
    fused_launches = ctx.launches - n0
    prog_b = opt_b.compile(grads_b, ctx, fused=False)
    numpy_step(g_steps[2])
    assert len(prog_a.calls) == 1 + 2, len(prog_a.calls)  # one call (two launches for 36 tensors), t + 1 and its copy
    assert len(prog_b.calls) >= 6 * len(ADAM_SHAPES) + 2
    for step in range(3, 6):
        feed(ga, g_steps[step]); feed(gb, g_steps[step])
        if step == 5:
            prog_a.capture()
        prog_a.run()
        prog_b.run()
        numpy_step(g_steps[step])
        for i, (a, b) in enumerate(zip(pa, pb)):
            exact(a.value.numpy(), b.value.numpy(), f"step {step} value {i}")
            exact(opt_a.m_t[id(ga[i])].numpy(), opt_b.m_t[id(gb[i])].numpy(), f"step {step} first moment {i}")
            exact(opt_a.v_t[id(ga[i])].numpy(), opt_b.v_t[id(gb[i])].numpy(), f"step {step} second moment {i}")
        exact(opt_a.t.numpy(), opt_b.t.numpy(), "step counter")
    prog_a.release_graph()
    for i, a in enumerate(pa):
        close(a.value.numpy(), w[i], 1e-4, f"value {i} vs float64")
        close(opt_a.v_t[id(ga[i])].numpy(), v[i], 2e-6, f"second moment {i} vs float64")  # 1 - beta2 formed in double would be 1.3e-5 off
    close(opt_a.t.numpy(), np.array([t]), 1e-6, "step counter vs float64")
    assert fused_launches <= 4

    # the entry point validates everything before it launches
    lib = ctx._lib
    from sage_amd import abi
    import ctypes as C
    one = lambda x: (abi.sg_tensor * 1)(x.c())
    hyper = abi.sg_adam_hyper(1e-2, 0.9, 0.999, OMB1, OMB2, 1e-8, 0.0)
    step_t = opt_a.t.c()
    small, big = pa[1].value, pa[2].value
    before = small.numpy().copy()
    with pytest.raises(abi.ShapeError):
        ctx.check(lib.sg_adam_update(ctx.handle, 1, one(small), one(big), one(small), one(small), C.byref(step_t), C.byref(hyper)))
    with pytest.raises(abi.ShapeError):  # step must be a single element
        ctx.check(lib.sg_adam_update(ctx.handle, 1, one(small), one(small), one(small), one(small), C.byref(big.c()), C.byref(hyper)))
    with pytest.raises(abi.DTypeError):
        idx = S.Tensor.from_numpy(ctx, np.zeros(3, np.int32))
        ctx.check(lib.sg_adam_update(ctx.handle, 1, one(small), one(idx), one(small), one(small), C.byref(step_t), C.byref(hyper)))
    exact(small.numpy(), before, "failed calls change nothing")
    assert lib.sg_adam_update(ctx.handle, 0, None, None, None, None, C.byref(step_t), C.byref(hyper)) == 0
