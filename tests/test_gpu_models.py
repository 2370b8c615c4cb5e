"""Model-level parity: BERT (models/bert.rs) and ResNet-18 (models/resnet.rs) through the HIP path
against the CPU oracle's op-for-op re-composition, and against an independent torch-CPU restatement.
Tolerance rel 1e-3 (end-to-end model output)."""
import numpy as np
import pytest

import sage_amd as S
from oracle import oracle as O
from sage_amd import var as V
from sage_amd.bert import Bert, BertConfig, BertLayer
from sage_amd.layers import load_params
from sage_amd.resnet import ResNet, ResNetConfig
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


def bert_layer_params(rng, e, hdim, per_feature):
    n = e if per_feature else 1
    w = lambda i, o: (rng.standard_normal((i, o)) * 0.05).astype(np.float32)
    v = lambda k: (rng.standard_normal((k,)) * 0.1).astype(np.float32)
    ln = lambda: ((1.0 + 0.1 * rng.standard_normal((n,))).astype(np.float32), (0.1 * rng.standard_normal((n,))).astype(np.float32))
    p = {"wk": w(e, e), "bk": v(e), "wq": w(e, e), "bq": v(e), "wv": w(e, e), "bv": v(e), "wo": w(e, e), "bo": v(e)}
    p["ln1_g"], p["ln1_b"] = ln()
    p["w1"], p["b1"], p["w2"], p["b2"] = w(e, hdim), v(hdim), w(hdim, e), v(e)
    p["ln2_g"], p["ln2_b"] = ln()
    return p


def layer_param_list(p):
    # BertLayer.params(): key, query, value, dense, norm ; ffn dense1, dense2 ; norm
    return [p["wk"], p["bk"], p["wq"], p["bq"], p["wv"], p["bv"], p["wo"], p["bo"], p["ln1_g"], p["ln1_b"],
            p["w1"], p["b1"], p["w2"], p["b2"], p["ln2_g"], p["ln2_b"]]


def torch_bert_layer(x, mask, p, heads, act, eps):
    import torch
    as_tensor = torch.is_tensor(x)  # tensors pass through (autograd use); arrays are converted
    t = lambda a: a if torch.is_tensor(a) else torch.from_numpy(np.asarray(a)).double()
    x = t(x)
    n, l, e = x.shape
    d = e // heads
    lin = lambda h, w, b: h @ t(w) + t(b)
    sep = lambda h: h.view(n, l, heads, d).transpose(1, 2)
    q, k, v = sep(lin(x, p["wq"], p["bq"])), sep(lin(x, p["wk"], p["bk"])), sep(lin(x, p["wv"], p["bv"]))
    s = q @ k.transpose(-1, -2) / np.sqrt(d) + (1.0 - t(mask).view(n, 1, 1, l)) * -1e5
    a = torch.softmax(s, -1) @ v
    a = a.transpose(1, 2).reshape(n, l, e)

    def lnorm(h, g, b):
        m = h.mean(-1, keepdim=True)
        var = (h * h).mean(-1, keepdim=True) - m * m
        return (h - m) / torch.sqrt(var + eps) * t(g) + t(b)

    h1 = lnorm(lin(a, p["wo"], p["bo"]) + x, p["ln1_g"], p["ln1_b"])
    u = lin(h1, p["w1"], p["b1"])
    u = torch.relu(u) if act == "relu" else 0.5 * u * (1 + torch.erf(u / np.sqrt(2.0)))
    out = lnorm(lin(u, p["w2"], p["b2"]) + h1, p["ln2_g"], p["ln2_b"])
    return out if as_tensor else out.numpy()


@pytest.mark.parametrize("reference_exact", [True, False], ids=["reference_exact", "gelu_config"])
@pytest.mark.parametrize("fused", [True, False], ids=["fused", "unfused"])
def test_bert_layer(ctx, reference_exact, fused):
    """BertLayer::pass (bert.rs:199-203) at n=2, l=24, e=64, 4 heads, ffn 160."""
    say("bert layer", reference_exact, fused)
    V.set_fusion(fused)
    rng = np.random.default_rng(3)
    n, l, e, heads, hdim = 2, 24, 64, 4, 160
    cfg = BertConfig(e, 100, 64, hdim, 1, heads, 1e-12, 0.1, 2)
    p = bert_layer_params(rng, e, hdim, per_feature=not reference_exact)
    x = rng.standard_normal((n, l, e)).astype(np.float32)
    mask = np.ones((n, l), np.float32)
    mask[1, 17:] = 0.0
    layer = BertLayer(cfg, reference_exact)
    load_params(ctx, layer, layer_param_list(p))
    n0 = ctx.launches
    y = layer.pass_(dev(ctx, x), dev(ctx, mask)).eval(ctx).numpy()
    launches = ctx.launches - n0
    say("launches", launches)
    act = "relu" if reference_exact else "gelu"
    eps = 1e-5 if reference_exact else 1e-12
    yo = O.bert_layer(ht(x), ht(mask), {k: ht(v) for k, v in p.items()}, heads, act, eps).numpy()
    close(y, yo, REL_GEMM, "vs oracle")
    close(y, torch_bert_layer(x, mask, p, heads, act, eps), REL_GEMM, "vs torch float64")
    if fused:
        assert launches <= 14, launches


def test_bert_model_reference_exact(ctx):
    """Bert::pass (bert.rs:72-81): embeddings -> 2 layers -> token 1 -> Dense."""
    say("bert model")
    rng = np.random.default_rng(5)
    cfg = BertConfig(32, 50, 40, 64, 2, 2, 0.0, 0.0, 3)
    n, l = 3, 12
    model = Bert(cfg, reference_exact=True)
    arrays = [(rng.standard_normal((50, 32))).astype(np.float32), rng.standard_normal((40, 32)).astype(np.float32),
              np.ones(1, np.float32), np.ones(1, np.float32)]
    layers = []
    for _ in range(2):
        p = bert_layer_params(rng, 32, 64, per_feature=False)
        layers.append(p)
        arrays += layer_param_list(p)
    wc, bc = (rng.standard_normal((32, 3)) * 0.1).astype(np.float32), np.zeros(3, np.float32)
    arrays += [wc, bc]
    load_params(ctx, model, arrays)
    ids = rng.integers(0, 50, (n, l)).astype(np.int32)
    mask = np.ones((n, l), np.float32)
    y = model.pass_(dev(ctx, ids), dev(ctx, mask), ctx).eval(ctx).numpy()
    po = {"word_emb": ht(arrays[0]), "pos_emb": ht(arrays[1]), "emb_g": ht(arrays[2]), "emb_b": ht(arrays[3]),
          "layers": [{k: ht(v) for k, v in p.items()} for p in layers], "wc": ht(wc), "bc": ht(bc)}
    yo = O.bert_forward(ht(ids.view(np.uint32).astype(np.uint32)), ht(mask), po, 2).numpy()
    assert y.shape == (n, 3)
    close(y, yo, REL_GEMM, "bert vs oracle")


def resnet_arrays(rng, chan_in, classes):
    """Parameters in ResNet.params() order + the oracle's dict form.  Kaiming-normal filters
    (std = sqrt(1/fan_in), tensor/init.rs:27-50), zero biases (layers.rs:373-381)."""
    def conv(kh, kw, ci, co):
        fan_in = kw * ci * co  # [d0=KH, d1=KW, rest=C*OC] -> fan_in = d1 * prod(rest)
        return (rng.standard_normal((kh, kw, ci, co)) * np.sqrt(1.0 / fan_in) * 4).astype(np.float32)
    arrays, blocks = [], []
    w0 = conv(7, 7, chan_in, 64)
    arrays += [w0, np.zeros(64, np.float32)]
    inp, out = 64, 64
    for i in range(4):
        stride = 1 if i == 0 else 2
        ip = inp
        for b in range(2):
            s = stride if b == 0 else 1
            blk = {"stride": s, "w1": conv(3, 3, ip, out), "b1": (rng.standard_normal(out) * 0.05).astype(np.float32),
                   "w2": conv(3, 3, out, out), "b2": (rng.standard_normal(out) * 0.05).astype(np.float32)}
            arrays += [blk["w1"], blk["b1"], blk["w2"], blk["b2"]]
            if s != 1 or ip != out:
                blk["wd"], blk["bd"] = conv(1, 1, ip, out), np.zeros(out, np.float32)
                arrays += [blk["wd"], blk["bd"]]
            blocks.append(blk)
            ip = out
        inp = out
        out *= 2
    wfc = (rng.standard_normal((512, classes)) * 0.05).astype(np.float32)
    bfc = np.zeros(classes, np.float32)
    arrays += [wfc, bfc]
    return arrays, {"w0": w0, "b0": arrays[1], "blocks": blocks, "wfc": wfc, "bfc": bfc}


@pytest.mark.parametrize("fused", [True, False], ids=["fused", "unfused"])
def test_resnet18(ctx, fused):
    """ResNet::new(d18(1,10)) (resnet.rs:75-104) on [3,28,28,1]."""
    say("resnet18", fused)
    V.set_fusion(fused)
    rng = np.random.default_rng(4)
    arrays, po = resnet_arrays(rng, 1, 10)
    model = ResNet(ResNetConfig.d18(1, 10))
    load_params(ctx, model, arrays)
    x = rng.uniform(0, 1, (3, 28, 28, 1)).astype(np.float32)
    n0 = ctx.launches
    y = model.pass_(dev(ctx, x)).eval(ctx).numpy()
    say("launches", ctx.launches - n0)
    conv = lambda d: {k: (ht(v) if isinstance(v, np.ndarray) else v) for k, v in d.items()}
    pod = {"w0": ht(po["w0"]), "b0": ht(po["b0"]), "blocks": [conv(b) for b in po["blocks"]], "wfc": ht(po["wfc"]), "bfc": ht(po["bfc"])}
    yo = O.resnet18_forward(ht(x), pod).numpy()
    assert y.shape == (3, 10)
    close(y, yo, REL_GEMM, "resnet vs oracle")


@pytest.mark.parametrize("model", ["bert_layer", "resnet18"])
def test_program_graph_replay(ctx, model):
    """A compiled Program replayed as a HIP graph: several replays, with new input values, eager runs and
    synchronisations between them, each compared with the eager result for the same input."""
    say("graph replay", model)
    rng = np.random.default_rng(11)
    if model == "bert_layer":
        n, l, e, heads, hdim = 2, 64, 128, 2, 256
        p = bert_layer_params(rng, e, hdim, per_feature=True)
        layer = BertLayer(BertConfig(e, 100, 512, hdim, 1, heads, 1e-12, 0.1, 2), reference_exact=False)
        load_params(ctx, layer, layer_param_list(p))
        xs = [rng.standard_normal((n, l, e)).astype(np.float32) for _ in range(3)]
        xt = S.Tensor.from_numpy(ctx, xs[0])
        out = layer.pass_(S.Var.new(xt), dev(ctx, np.ones((n, l), np.float32)))
    else:
        arrays, _ = resnet_arrays(rng, 1, 10)
        net = ResNet(ResNetConfig.d18(1, 10))
        load_params(ctx, net, arrays)
        xs = [rng.uniform(0, 1, (16, 28, 28, 1)).astype(np.float32) for _ in range(3)]
        xt = S.Tensor.from_numpy(ctx, xs[0])
        out = net.pass_(S.Var.new(xt))
    prog = S.Program(ctx, [out])
    eager = []
    for x in xs:
        xt.copy_from_numpy(x)
        eager.append(prog.run_eager()[0].numpy().copy())
    assert not np.array_equal(eager[0], eager[1])
    prog.capture()
    try:
        for rep in range(2):
            for x, want in zip(xs, eager):
                xt.copy_from_numpy(x)
                got = prog.run()[0].numpy()
                exact(got, want, f"graph replay {rep} vs eager")
                ctx.sync()
                xt.copy_from_numpy(xs[0])
                exact(prog.run_eager()[0].numpy(), eager[0], "eager between replays")
    finally:
        prog.release_graph()


def test_memory_capped_evaluation_evicts_and_recomputes(ctx):
    """Program::exec under a memory cap (session.rs:259-325): the same BERT layers evaluated in a context whose
    capacity is a fraction of what the uncapped run holds at its peak.  Intermediates are dropped after their last
    use, and when an allocation still does not fit, retained tensors are evicted and recomputed on demand; the
    result is bit-identical and the allocator never hands out more than the cap."""
    say("capped evaluation")
    rng = np.random.default_rng(21)
    n, l, e, heads, hdim, nlayers = 4, 128, 256, 4, 384, 8
    layers_p = [bert_layer_params(rng, e, hdim, per_feature=True) for _ in range(nlayers)]
    x = rng.standard_normal((n, l, e)).astype(np.float32)
    mask = np.ones((n, l), np.float32)

    def run(c):
        h = S.Var.new(S.Tensor.from_numpy(c, x))
        m = S.Var.new(S.Tensor.from_numpy(c, mask))
        outs = []
        for p in layers_p:
            layer = BertLayer(BertConfig(e, 100, 512, hdim, 1, heads, 1e-12, 0.1, 2), reference_exact=False)
            load_params(c, layer, layer_param_list(p))
            h = layer.pass_(h, m)
            outs.append(h)
        # every layer's output has a late consumer: each must survive until then or be recomputed
        y = outs[-1]
        for o in outs[:-1]:
            y = y + o
        ev = V._Evaluator(c, [y])
        out = ev.get(y).numpy()
        # the reference's order (session.rs:300-310): smallest (exec_time + 1) / (size + 1) first; with issue times far
        # below a second that is largest first
        for sizes in ev.eviction_log:
            assert sizes == sorted(sizes, reverse=True), sizes
        return out, ev.evictions, c.mem_stats()

    fresh = S.Context(0)
    try:
        want, ev0, st0 = run(fresh)
    finally:
        fresh.close()
    assert ev0 == 0
    params_bytes = sum(a.nbytes for p in layers_p for a in p.values()) + x.nbytes + mask.nbytes
    act_peak = st0["peak"] - params_bytes  # what the uncapped run held besides parameters and inputs
    say("uncapped peak beyond parameters", act_peak, "bytes =", act_peak / (n * l * e * 4), "activations")
    results = []
    for frac in (0.8, 0.7, 0.6):
        cap = params_bytes + int(frac * act_peak)
        c = S.Context(0, capacity=cap)
        try:
            got, evictions, st = run(c)
        finally:
            c.close()
        exact(got, want, f"cap at {frac} of the uncapped peak")
        assert st["peak"] <= cap, (st, cap)
        say("cap", frac, "evictions", evictions, "peak", st["peak"])
        results.append(evictions)
    assert results[-1] > 0, "the tightest cap must have forced evictions"
    hopeless = S.Context(0, capacity=params_bytes + n * l * e * 4)
    try:
        with pytest.raises(S.abi.OutOfMemory):
            run(hopeless)
    finally:
        hopeless.close()


@pytest.mark.parametrize("name", ["densenet121", "mobilenetv2", "resnet50"])
def test_other_model_families_vs_oracle(ctx, name):
    """DenseNet (densenet.rs), MobileNetV2 (mobilenet.rs, with its dilation-0 3x3 stage) and the bottleneck ResNets
    (resnet.rs:178-243): parameters from the layers' own init, forward pass against the oracle's layer-by-layer
    evaluation of the same layer tree; fused and operator-by-operator evaluation agree."""
    from sage_amd.densenet import DenseNet, DenseNetConfig
    from sage_amd.mobilenet import MobileNetV2, MobileNetV2Config
    from tests import oracle_layers
    say("model", name)
    rng = np.random.default_rng(7)
    model = {"densenet121": lambda: DenseNet(DenseNetConfig.d121(3, 10)), "mobilenetv2": lambda: MobileNetV2(MobileNetV2Config(3, 10)),
             "resnet50": lambda: ResNet(ResNetConfig.d50(3, 10))}[name]()
    model.init(ctx, rng)
    for p in model.params():  # biases start at zero (layers.rs:233, 383): give them values so they are exercised
        if p.rank == 1:
            p.set(S.Tensor.from_numpy(ctx, (rng.standard_normal(p.extents) * 0.1).astype(np.float32)))
    x = rng.uniform(0, 1, (2, 32, 32, 3)).astype(np.float32)
    n0 = ctx.launches
    y = model.pass_(dev(ctx, x)).eval(ctx).numpy()
    fused = ctx.launches - n0
    yo = oracle_layers.forward(model, ht(x)).numpy()
    assert y.shape == (2, 10) and np.all(np.isfinite(y))
    close(y, yo, REL_GEMM, "fused vs oracle")
    V.set_fusion(False)
    n0 = ctx.launches
    y2 = model.pass_(dev(ctx, x)).eval(ctx).numpy()
    close(y2, yo, REL_GEMM, "operator by operator vs oracle")
    say("launches", fused, "fused,", ctx.launches - n0, "operator by operator")


def test_batch_norm_2d_function_and_layer(ctx):
    """batch_norm_2d (conv.rs:167-185): gamma * (x - mean) / sqrt(var + eps) + beta with per-channel
    statistics broadcast over [N,H,W,C]; BatchNorm2d (layers.rs:479-548) normalises with its running
    statistics, scalar gamma/beta and a hard-coded eps of 1e-05.  Against float64 and the oracle's maps."""
    from sage_amd.layers import BatchNorm2d
    say("batch_norm_2d")
    rng = np.random.default_rng(21)
    n, h, w, c = 3, 5, 7, 12
    x = rng.standard_normal((n, h, w, c)).astype(np.float32)
    mean = rng.standard_normal(c).astype(np.float32)
    var = rng.uniform(0.2, 3.0, c).astype(np.float32)
    for gshape in ((1,), (c,)):
        gamma = rng.uniform(0.5, 1.5, gshape).astype(np.float32)
        beta = rng.standard_normal(gshape).astype(np.float32)
        for eps in (1e-5, 0.1):
            n0 = ctx.launches
            y = V.batch_norm_2d(dev(ctx, x), dev(ctx, gamma), dev(ctx, beta), dev(ctx, mean), dev(ctx, var), eps).eval(ctx).numpy()
            assert ctx.launches - n0 == 2  # sqrt(var + eps) on [C], then one fused map over [N,H,W,C]
            ref = gamma.astype(np.float64) * (x.astype(np.float64) - mean) / np.sqrt(var.astype(np.float64) + np.float32(eps)) + beta
            close(y, ref, REL_MAP, f"batch_norm_2d gamma{gshape} eps {eps} vs float64")
            ex = [n, h, w, c]
            xc = O.binary("div", O.binary("sub", ht(x), ht(mean).expand(ex)), O.unary("sqrt", O.binary("add", ht(var), float(eps))).expand(ex))
            yo = O.binary("add", O.binary("mul", ht(gamma).expand(ex), xc), ht(beta).expand(ex)).numpy()
            exact(y, yo, "vs the oracle's maps (+,-,*,/,sqrt are exact)")
    say("BatchNorm2d layer")
    layer = BatchNorm2d(c, 0.5)  # the eps given here is ignored by the reference's pass
    layer.init(ctx, rng)
    y = layer.pass_(dev(ctx, x)).eval(ctx).numpy()
    close(y, (x.astype(np.float64) - 1.0) / np.sqrt(1.0 + np.float32(1e-5)) + 1.0, REL_MAP, "initial statistics (all ones)")
    layer.running_mean.set(S.Tensor.from_numpy(ctx, mean))
    layer.running_var.set(S.Tensor.from_numpy(ctx, var))
    layer.gamma.set(S.Tensor.from_numpy(ctx, np.array([1.25], np.float32)))
    layer.beta.set(S.Tensor.from_numpy(ctx, np.array([-0.5], np.float32)))
    y = layer.pass_(dev(ctx, x)).eval(ctx).numpy()
    close(y, 1.25 * (x.astype(np.float64) - mean) / np.sqrt(var.astype(np.float64) + np.float32(1e-5)) - 0.5, REL_MAP, "running statistics")
    assert [p.label for p in layer.params()] == ["batch_norm_2d.gamma", "batch_norm_2d.beta"]
