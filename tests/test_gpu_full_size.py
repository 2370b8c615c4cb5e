"""The five benchmark configurations at their full sizes.

Where the CPU oracle finishes in seconds the whole result is compared with it; where it would not,
size-independent properties are used instead: sampled entries against float64 dot products,
a row block against the oracle, and batch-slice invariance (the first sequences of a full batch must
equal a run on just those sequences, which the oracle can check)."""
import numpy as np
import pytest

import sage_amd as S
from oracle import oracle as O
from sage_amd import nn
from sage_amd import var as V
from sage_amd.bert import BertConfig, BertLayer
from sage_amd.layers import load_params
from sage_amd.resnet import ResNet, ResNetConfig
from tests.test_gpu_models import bert_layer_params, layer_param_list, resnet_arrays
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


def test_config1_softmax_cross_entropy_8192x1024(ctx):
    say("C1 softmax-CE [8192,1024]")
    rng = np.random.default_rng(1)
    x = rng.standard_normal((8192, 1024)).astype(np.float32)
    lab = rng.integers(0, 1024, (8192, 1)).astype(np.int32)
    y = nn.softmax_cross_entropy(dev(ctx, x), dev(ctx, lab)).eval(ctx).numpy()
    x64 = x.astype(np.float64)
    ref = -(x64[np.arange(8192), lab[:, 0]] - np.log(np.exp(x64).sum(1)))
    close(y, ref, REL_MAP, "fused vs float64")
    close(y, O.softmax_cross_entropy(ht(x), ht(lab.astype(np.uint32))).numpy(), REL_MAP, "fused vs oracle")
    V.set_fusion(False)
    close(nn.softmax_cross_entropy(dev(ctx, x), dev(ctx, lab)).eval(ctx).numpy(), ref, REL_MAP, "composed vs float64")
    assert np.all(y >= 0)


def test_config2_gemm_4096_bias(ctx):
    say("C2 GEMM 4096^3 + bias")
    rng = np.random.default_rng(2)
    n = 4096
    a = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    b = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    bias = rng.uniform(-1, 1, (n,)).astype(np.float32)
    n0 = ctx.launches
    y = (dev(ctx, a).matmul(dev(ctx, b)) + dev(ctx, bias)).eval(ctx).numpy()
    assert ctx.launches - n0 == 1
    ii, jj = rng.integers(0, n, 512), rng.integers(0, n, 512)
    ref = np.einsum("ik,ki->i", a[ii].astype(np.float64), b[:, jj].astype(np.float64)) + bias[jj]
    close(y[ii, jj], ref, REL_GEMM, "sampled entries vs float64")
    rows = np.arange(1000, 1016)
    close(y[rows], O.dense(ht(a[rows]), ht(b), ht(bias)).numpy(), REL_GEMM, "16-row block vs oracle")
    # a checksum of checksums: sum_j C[i,j] = A[i,:] . (B 1) + sum(bias)
    close(y.astype(np.float64).sum(1), a.astype(np.float64) @ b.astype(np.float64).sum(1) + bias.astype(np.float64).sum(), REL_GEMM, "row checksums")


@pytest.mark.parametrize("reference_exact", [True, False], ids=["reference_exact", "gelu_config"])
def test_config3_bert_layer_b32_s128(ctx, reference_exact):
    say("C3 BERT layer b32 s128 h768", reference_exact)
    rng = np.random.default_rng(3)
    n, l, e, heads, hdim = 32, 128, 768, 12, 3072
    p = bert_layer_params(rng, e, hdim, per_feature=not reference_exact)
    for k in p:
        if k.startswith("w"):
            p[k] = (p[k] * 0.4).astype(np.float32)  # ~N(0, 0.02)
    x = rng.standard_normal((n, l, e)).astype(np.float32)
    mask = np.ones((n, l), np.float32)
    layer = BertLayer(BertConfig(e, 100, 512, hdim, 1, heads, 1e-12, 0.1, 2), reference_exact)
    load_params(ctx, layer, layer_param_list(p))
    n0 = ctx.launches
    y = layer.pass_(dev(ctx, x), dev(ctx, mask)).eval(ctx).numpy()
    say("launches", ctx.launches - n0)
    act, eps = ("relu", 1e-5) if reference_exact else ("gelu", 1e-12)
    yo = O.bert_layer(ht(x), ht(mask), {k: ht(v) for k, v in p.items()}, heads, act, eps).numpy()
    close(y, yo, REL_GEMM, "vs oracle")


LAYER_KEYS = ["wk", "bk", "wq", "bq", "wv", "bv", "wo", "bo", "ln1_g", "ln1_b", "w1", "b1", "w2", "b2", "ln2_g", "ln2_b"]


def oracle_bert_params(arrays, layers, segments):
    """Host arrays in Bert.params() order -> the oracle's parameter dict."""
    it = iter(arrays)
    p = {"word_emb": ht(next(it)), "pos_emb": ht(next(it))}
    if segments:
        p["seg_emb"] = ht(next(it))
    p["emb_g"], p["emb_b"] = ht(next(it)), ht(next(it))
    p["layers"] = [{k: ht(next(it)) for k in LAYER_KEYS} for _ in range(layers)]
    p["wc"], p["bc"] = ht(next(it)), ht(next(it))
    assert next(it, None) is None
    return p


def worst(a, b):
    """max |a-b| / max(|b|, rms(b)): the figure `close` bounds, as a number to print."""
    a, b = a.astype(np.float64), b.astype(np.float64)
    return float(np.max(np.abs(a - b) / np.maximum(np.abs(b), np.sqrt(np.mean(b * b)))))


def as_uint(ids):
    return ht(ids.view(np.uint32))


@pytest.mark.parametrize("variant", ["config", "reference"])
def test_headline_bert_base_b32_s128_twelve_layers_end_to_end(ctx, variant):
    """The model bench.py times (same builder, same seed): BERT-base, 12 layers, vocab 30522, b32 x s128.
    Logits and the last encoder output against the oracle's op-for-op evaluation of Bert::pass
    (bert.rs:72-81, 128-139), within the end-to-end bound of rel 1e-3."""
    import bench
    say("headline BERT-base b32 s128, 12 layers, end to end:", variant)
    d = bench.build_bert(ctx, variant, 32, 128, 12, np.random.default_rng(5), detail=True)
    prog = S.Program(ctx, [d["logits"], d["hidden"]])
    logits, hidden = (t.numpy() for t in prog.outputs)
    say("launches per step", len(prog.calls))
    exact_variant = variant == "reference"
    po = oracle_bert_params(d["arrays"], 12, 0 if exact_variant else 2)
    act, eps, cls = ("relu", 1e-5, 1) if exact_variant else ("gelu", 1e-12, 0)
    seg = None if d["segment_ids"] is None else as_uint(d["segment_ids"])
    lo, ho = O.bert_forward(as_uint(d["ids"]), ht(d["mask"]), po, 12, act, eps, cls, seg, return_hidden=True)
    lo, ho = lo.numpy(), ho.numpy()
    say(f"worst error / tolerance scale: logits {worst(logits, lo):.3e}, last encoder output {worst(hidden, ho):.3e} (bound 1e-3)")
    assert logits.shape == (32, 2) and hidden.shape == (32, 128, 768)
    close(hidden, ho, REL_GEMM, "last encoder output vs oracle")
    close(logits, lo, REL_GEMM, "logits vs oracle")
    # the replayed program (what the benchmark times) gives the same bits as its first evaluation
    prog.run()
    assert np.array_equal(prog.outputs[0].numpy(), logits)


def test_config5_full_bert_base_b64_s512_segments(ctx):
    """Configuration 5 as written: 12 layers, b64 x s512, vocab 30522, position and segment embeddings,
    classifier on the [CLS] token.  The oracle cannot run 32768 tokens through 12 layers in seconds, so:
    the embedding gather at [32768,768] (stride-0 index, layers.rs:430-446) is bit-exact against numpy
    fancy indexing, the first two sequences of the full batch equal a batch-of-2 run, that run equals the
    oracle end to end, and everything is finite."""
    from sage_amd.bert import Bert
    say("C5 full BERT-base b64 s512 with segment embeddings")
    rng = np.random.default_rng(55)
    n, l, layers = 64, 512, 12
    cfg = BertConfig.base()
    model = Bert(cfg, reference_exact=False, segments=2)
    arrays = []
    for p in model.params():
        name = p.label or ""
        if "layer_norm.gamma" in name:
            a = (1.0 + 0.1 * rng.standard_normal(p.extents)).astype(np.float32)
        elif "layer_norm.beta" in name or name.endswith(".bias"):
            a = (0.05 * rng.standard_normal(p.extents)).astype(np.float32)
        else:
            a = (rng.standard_normal(p.extents) * 0.02).astype(np.float32)
        arrays.append(a)
    load_params(ctx, model, arrays)
    ids = rng.integers(0, cfg.num_vocabs, (n, l)).astype(np.int32)
    ids[0, :4] = [0, cfg.num_vocabs - 1, 0, cfg.num_vocabs - 1]  # both ends of the table
    seg = rng.integers(0, 2, (n, l)).astype(np.int32)
    mask = np.ones((n, l), np.float32)
    mask[1, 300:] = 0.0
    mask[63, 17:] = 0.0

    say("embedding gather [32768,768] from the 30522-row table")
    we = model.embedding.word_emb.pass_(dev(ctx, ids)).eval(ctx).numpy()
    assert np.array_equal(we, arrays[0][ids])
    se = model.embedding.seg_emb.pass_(dev(ctx, seg)).eval(ctx).numpy()
    assert np.array_equal(se, arrays[2][seg])
    e_sum = (model.embedding.word_emb.pass_(dev(ctx, ids)) + model.embedding.pos_emb.pass_(dev(ctx, np.arange(l, dtype=np.uint32)))
             + model.embedding.seg_emb.pass_(dev(ctx, seg))).eval(ctx).numpy()
    assert np.array_equal(e_sum, (arrays[0][ids] + arrays[1][:l]) + arrays[2][seg])

    def run(sl):
        ids_v, mask_v, seg_v = dev(ctx, ids[sl]), dev(ctx, mask[sl]), dev(ctx, seg[sl])
        hidden = model.encode(model.embedding.pass_(ids_v, ctx, seg_v), mask_v)
        out = V.evaluate_fresh(ctx, [model.classify(hidden), hidden])
        return out[0].numpy(), out[1].numpy()

    say("full batch")
    logits_full, hidden_full = run(slice(0, n))
    assert logits_full.shape == (n, 2) and hidden_full.shape == (n, l, 768)
    assert np.all(np.isfinite(logits_full)) and np.all(np.isfinite(hidden_full))
    say("batch of 2 and batch-slice invariance")
    logits_two, hidden_two = run(slice(0, 2))
    close(hidden_full[:2], hidden_two, REL_GEMM, "first two sequences of the full batch vs a batch of two")
    close(logits_full[:2], logits_two, REL_GEMM, "logits, batch-slice invariance")
    logits_last, hidden_last = run(slice(62, 64))
    close(hidden_full[62:], hidden_last, REL_GEMM, "last two sequences (one heavily masked)")
    say("batch of 2 vs the oracle, 12 layers end to end")
    po = oracle_bert_params(arrays, layers, 2)
    lo, ho = O.bert_forward(as_uint(ids[:2]), ht(mask[:2]), po, 12, "gelu", 1e-12, 0, as_uint(seg[:2]), return_hidden=True)
    say(f"worst error / tolerance scale: logits {worst(logits_two, lo.numpy()):.3e}, hidden {worst(hidden_two, ho.numpy()):.3e} (bound 1e-3)")
    close(hidden_two, ho.numpy(), REL_GEMM, "batch of 2 vs oracle: last encoder output")
    close(logits_two, lo.numpy(), REL_GEMM, "batch of 2 vs oracle: logits")
    # every layer ends in a LayerNorm: undoing the last one's affine part leaves rows of mean 0, variance 1
    g, b = arrays[-4].astype(np.float64), arrays[-3].astype(np.float64)
    z = (hidden_full.astype(np.float64) - b) / g
    assert np.abs(z.mean(-1)).max() < 1e-3
    close(z.var(-1), np.ones(z.shape[:2]), REL_GEMM, "rows normalised")


def test_config4_resnet18_b128(ctx):
    say("C4 ResNet-18 b128 28x28x1")
    rng = np.random.default_rng(4)
    arrays, po = resnet_arrays(rng, 1, 10)
    model = ResNet(ResNetConfig.d18(1, 10))
    load_params(ctx, model, arrays)
    x = rng.uniform(0, 1, (128, 28, 28, 1)).astype(np.float32)
    y = model.pass_(dev(ctx, x)).eval(ctx).numpy()
    conv = lambda d: {k: (ht(v) if isinstance(v, np.ndarray) else v) for k, v in d.items()}
    pod = {"w0": ht(po["w0"]), "b0": ht(po["b0"]), "blocks": [conv(b) for b in po["blocks"]], "wfc": ht(po["wfc"]), "bfc": ht(po["bfc"])}
    close(y, O.resnet18_forward(ht(x), pod).numpy(), REL_GEMM, "vs oracle")


def test_config5_bert_layer_b64_s512_batch_slice(ctx):
    say("C5 BERT layer b64 s512: first 2 sequences of the full batch == a batch of 2 == oracle")
    rng = np.random.default_rng(5)
    n, l, e, heads, hdim = 64, 512, 768, 12, 3072
    p = bert_layer_params(rng, e, hdim, per_feature=True)
    for k in p:
        if k.startswith("w"):
            p[k] = (p[k] * 0.4).astype(np.float32)
    x = rng.standard_normal((n, l, e)).astype(np.float32)
    mask = np.ones((n, l), np.float32)
    mask[1, 400:] = 0.0
    layer = BertLayer(BertConfig(e, 100, 512, hdim, 1, heads, 1e-12, 0.1, 2), reference_exact=False)
    load_params(ctx, layer, layer_param_list(p))
    y_full = layer.pass_(dev(ctx, x), dev(ctx, mask)).eval(ctx).numpy()
    y_two = layer.pass_(dev(ctx, x[:2]), dev(ctx, mask[:2])).eval(ctx).numpy()
    close(y_full[:2], y_two, REL_GEMM, "batch-slice invariance")
    yo = O.bert_layer(ht(x[:2]), ht(mask[:2]), {k: ht(v) for k, v in p.items()}, heads, "gelu", 1e-12).numpy()
    close(y_two, yo, REL_GEMM, "batch of 2 vs oracle")
    assert np.all(np.isfinite(y_full))
    # the layer ends in a layer norm: undoing its affine part leaves rows of mean 0 and variance 1
    z = (y_full.astype(np.float64) - p["ln2_b"]) / p["ln2_g"]
    assert np.abs(z.mean(-1)).max() < 1e-3
    close(z.var(-1), np.ones(z.shape[:2]), REL_GEMM, "rows normalised")


def test_streamed_maps_at_full_size_are_exact(ctx):
    """Maps whose operands total more than the streaming threshold take non-temporal loads and stores:
    the three-input (g + bias) + x map of a BERT layer at [4096, 3072] (151 MB) and a strided-operand
    map of the same size are bit-exact against numpy, the exp(x - c) map of config 1 (67 MB) matches the
    oracle; the same expressions on a small tensor (regular accesses) agree with their full-size rows."""
    rng = np.random.default_rng(12)
    m, n = 4096, 3072
    g = rng.standard_normal((m, n)).astype(np.float32)
    x = rng.standard_normal((m, n)).astype(np.float32)
    bias = rng.standard_normal((n,)).astype(np.float32)
    say("streamed (g+bias)+x", (m, n))
    y = ((dev(ctx, g) + dev(ctx, bias)) + dev(ctx, x)).eval(ctx).numpy()
    assert np.array_equal(y, (g + bias) + x)
    small = ((dev(ctx, g[:8]) + dev(ctx, bias)) + dev(ctx, x[:8])).eval(ctx).numpy()
    assert np.array_equal(small, y[:8])
    say("streamed map with a transposed operand", (n, m))
    yt = (dev(ctx, g).transpose(0, 1) * 2.0 + dev(ctx, x.T.copy())).eval(ctx).numpy()
    assert np.array_equal(yt, g.T * np.float32(2.0) + x.T)
    say("streamed exp(x - c)", (8192, 1024))
    lg = rng.standard_normal((8192, 1024)).astype(np.float32)
    c = lg.max(1, keepdims=True)
    e = (dev(ctx, lg) - dev(ctx, c)).exp().eval(ctx).numpy()
    close(e[:64], O.unary("exp", O.binary("sub", ht(lg[:64]), ht(c[:64]).expand([64, 1024]))).numpy(), REL_MAP, "rows vs oracle")
    assert np.all(e <= 1.0) and np.all(e.max(1) == 1.0)


def test_config5_bert_b64_s512_under_a_memory_cap():
    """Program::exec's memory behaviour (session.rs:259-330) on the model of configuration 5 (12 layers, b64 x s512, vocab
    30522) in contexts whose capacity is below what an uncapped evaluation holds at its peak.

    (1) The forward pass alone: intermediates die with their last consumer, so the activation peak is one operator's
    working set (the second FFN product reads [32768,3072] and the [32768,768] residual and writes [32768,768]: 0.6 GB).
    Under 0.9 of the peak it evicts retained tensors and recomputes them; under 0.8 that one operator's own operands no
    longer fit and the evaluation fails with OutOfMemory, as the reference's would (it can only evict what the running
    operator does not use, session.rs:294-325).
    (2) The same model with every encoder layer's output kept alive by a late consumer (what a backward pass does to the
    activations, the case the reference's eviction is for): capacity = parameters + 0.6 x the uncapped activation peak.
    Every result is bit-identical to the uncapped one and the allocator never exceeds the capacity."""
    import bench
    from sage_amd import var as V

    def run(capacity, retain):
        c = S.Context(0, capacity=capacity) if capacity else S.Context(0)
        try:
            d = bench.build_bert(c, "config", 64, 512, 12, np.random.default_rng(5), detail=True)
            model = d["model"]
            if not retain:
                targets = [d["logits"]]
            else:
                ids, mask, seg = (S.Var.new(S.Tensor.from_numpy(c, d[k])) for k in ("ids", "mask", "segment_ids"))
                h = model.embedding.pass_(ids, c, seg)
                outs = []
                for layer in model.layers:
                    h = layer.pass_(h, mask)
                    outs.append(h)
                # every layer's output is read once more, one at a time, after the last layer has run: the mean over its tokens
                late = [o.mean(1, False) for o in outs]
                targets = [model.classify(outs[-1])] + late
            ev = V._Evaluator(c, targets)
            out = np.concatenate([ev.get(t).numpy().ravel() for t in targets])
            return out, ev.evictions, c.mem_stats(), sum(a.nbytes for a in d["arrays"])
        finally:
            c.close()

    for retain in (False, True):
        say("C5 under a cap, layer outputs retained:", retain)
        want, ev0, st0, params_bytes = run(0, retain)
        assert ev0 == 0 and np.all(np.isfinite(want))
        act_peak = st0["peak"] - params_bytes
        say("uncapped activation peak", act_peak, "bytes =", round(act_peak / (64 * 512 * 768 * 4), 2), "x [32768,768]")
        frac = 0.6 if retain else 0.9
        cap = params_bytes + int(frac * act_peak)
        got, evictions, st, _ = run(cap, retain)
        say("cap", frac, "evictions", evictions, "peak", st["peak"], "of", cap)
        exact(got, want, f"capacity = parameters + {frac} x activation peak")
        assert st["peak"] <= cap and evictions > 0
        if not retain:
            with pytest.raises(S.abi.OutOfMemory):
                run(params_bytes + int(0.8 * act_peak), retain)
