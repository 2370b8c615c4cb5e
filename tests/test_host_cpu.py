"""CPU-only checks: the stride algebra, the C-ABI library (loads, exports every declared symbol),
the run-time kernel generator (source + gfx950 compile, no GPU needed) and the rule that the
product never reaches into the oracle."""
import ctypes as C
import os
import re
import subprocess

import numpy as np
import pytest

from sage_amd import abi
from sage_amd.shape import Shape, ShapeError, default_strides, infer_extents, norm_axes, norm_axis, union

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ------------------------------------------------------------------ shape.rs:707-870
def test_axis():
    assert norm_axis(-3, 3) == 0 and norm_axis(-2, 3) == 1 and norm_axis(0, 3) == 0 and norm_axis(1, 3) == 1
    for a, b in ((0, 0), (-4, 3), (4, 4)):
        with pytest.raises(ShapeError):
            norm_axis(a, b)
    assert norm_axes([-3, -2, -1, 0, 1, 2], 3) == [0, 1, 2, 0, 1, 2]
    with pytest.raises(ShapeError):
        norm_axes([-4, -2, -1, 0, 1, 2], 3)


def test_extents():
    assert infer_extents([2, 3, 4], 0) == [2, 3, 4]
    assert infer_extents([2, 3, 4], 24) == [2, 3, 4]
    assert infer_extents([-1, 3, 4], 24) == [2, 3, 4]
    assert infer_extents([2, -1, 4], 24) == [2, 3, 4]
    assert infer_extents([2, 3, -1], 24) == [2, 3, 4]
    for ext, size in (([1, 3, -4], 24), ([1, 0, 4], 24), ([1, 3, 4], 24), ([1, 3, 4], 23), ([1, 3, 4], 25),
                      ([-1, -1, 4], 24), ([-1, 3, 4], 0), ([-1, 3, 4], 25)):
        with pytest.raises(ShapeError):
            infer_extents(ext, size)


def test_union():
    assert union([1, 3, 4], [1, 3, 4]) == [1, 3, 4]
    assert union([5, 6, 1, 3, 4], [1, 3, 4]) == [5, 6, 1, 3, 4]
    assert union([5, 6, 1, 3, 4], [7, 3, 4]) == [5, 6, 7, 3, 4]
    assert union([1, 2, 1, 2, 1, 2], [2, 1, 2, 1, 2, 1]) == [2, 2, 2, 2, 2, 2]
    with pytest.raises(ShapeError):
        union([2, 3], [4, 3])


def test_shape_algebra_against_numpy():
    """Every layout method against numpy's own stride arithmetic on a real array."""
    a = np.arange(2 * 3 * 4 * 5, dtype=np.float32).reshape(2, 3, 4, 5)
    flat = a.reshape(-1)

    def realise(sh):
        return np.array(np.lib.stride_tricks.as_strided(flat[sh.offset:], sh.extents, [s * 4 for s in sh.strides]))

    s = Shape(a.shape)
    assert s.strides == [60, 20, 5, 1] == default_strides(a.shape) and s.has_default_strides()
    assert np.array_equal(realise(s.permute([2, 0, 3, 1])), a.transpose(2, 0, 3, 1))
    assert np.array_equal(realise(s.swap(1, 3)), a.swapaxes(1, 3))
    assert np.array_equal(realise(s.select_range(1, 2, 2)), a[:, :, 1:3])
    assert np.array_equal(realise(s.select(2, 1)), a[:, 2])
    assert np.array_equal(realise(s.select_range(0, 0, 1).remove(1).insert(0)), a[None, :, 0])
    e = Shape([3, 1, 5]).expand([2, 1, 3, 9, 5])  # the example in shape.rs:248-249
    assert e.extents == [2, 1, 3, 9, 5] and e.strides == [0, 0, 5, 0, 1]
    with pytest.raises(ShapeError):
        Shape([3, 2]).expand([3, 4])
    # has_default_strides ignores the offset (shape.rs:134-143); insert() gives stride 0 (shape.rs:190-195)
    assert s.select_range(1, 1, 0).has_default_strides()
    assert not Shape([4]).insert(1).has_default_strides()
    for i in range(s.size()):
        t = s.permute([3, 1, 0, 2])
        assert flat[t.translate_default(i)] == a.transpose(3, 1, 0, 2).reshape(-1)[i]
    inner, outer = s.extract([1, 3], True)
    assert inner.extents == [3, 5] and inner.strides == [20, 1] and outer.extents == [2, 4] and outer.strides == [60, 5]
    assert Shape([2, 3]).is_contiguous() and not Shape([2, 3], [6, 1]).is_contiguous()
    assert not Shape([2, 3]).expand([4, 2, 3]).is_bijective()


# ------------------------------------------------------------------ the C-ABI library
def declared_symbols():
    text = open(os.path.join(ROOT, "include", "sage_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sg_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_symbols()
    assert len(names) >= 35
    lib = abi.lib()  # raises if the library is missing or a prototype has no symbol
    out = subprocess.check_output(["nm", "-D", "--defined-only", abi.LIB_PATH], text=True)
    exported = set(re.findall(r" T (sg_[a-z0-9_]+)", out))
    assert set(names) <= exported, sorted(set(names) - exported)
    assert set(names) == set(abi.PROTOTYPES), (sorted(set(names) ^ set(abi.PROTOTYPES)))
    for n in names:
        assert getattr(lib, n) is not None


def test_struct_layout_matches_header():
    assert C.sizeof(abi.sg_tensor) == 8 + 4 + 4 + 8 * 8 + 8 * 8 + 8
    assert C.sizeof(abi.sg_expr) == 16
    assert abi.sg_tensor.offset.offset == 144 and abi.sg_tensor.strides.offset == 80


def test_no_context_without_gpu_is_an_error_not_a_fallback():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    h = C.c_void_p()
    assert abi.lib().sg_ctx_create(0, 0, C.byref(h)) == abi.ERR_DEVICE and not h.value


def test_product_does_not_touch_the_oracle():
    for d, _, files in os.walk(os.path.join(ROOT, "sage_amd")):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(d, f)).read()
                assert "oracle" not in text.replace("CPU oracle", ""), f


# ------------------------------------------------------------------ run-time kernel generator
def desc(extents, strides=None, offset=0, dtype=abi.FLOAT):
    t = abi.sg_tensor()
    t.base = None
    t.dtype = dtype
    t.rank = len(extents)
    st = default_strides(extents) if strides is None else strides
    for i, (e, s) in enumerate(zip(extents, st)):
        t.extents[i], t.strides[i] = e, s
    t.offset = offset
    return t


def prog(*items):
    arr = (abi.sg_expr * len(items))()
    for i, (k, o, d, b) in enumerate(items):
        arr[i].kind, arr[i].op, arr[i].dtype, arr[i].bits = k, o, d, b
    return arr, len(items)


def source(items, ins, out):
    arr, n = prog(*items)
    buf = C.create_string_buffer(1 << 16)
    dt = C.c_int32(-1)
    inarr = (abi.sg_tensor * max(1, len(ins)))(*ins)
    rc = abi.lib().sg_map_source(None, arr, n, inarr, len(ins), C.byref(out), buf, len(buf), C.byref(dt))
    return rc, buf.value.decode(), dt.value


def compiles(src):
    log = C.create_string_buffer(1 << 14)
    rc = abi.lib().sg_map_compile_only(src.encode(), log, len(log))
    assert rc == abi.OK, log.value.decode()


INP = lambda i: (abi.EXPR_INPUT, i, 0, 0)
UN = lambda n: (abi.EXPR_UNARY, abi.U[n], 0, 0)
BIN = lambda n: (abi.EXPR_BINARY, abi.B[n], 0, 0)
LITF = lambda v: (abi.EXPR_LITERAL, 0, abi.FLOAT, int(np.float32(v).view(np.uint32)))
COND = (abi.EXPR_TERNARY, 0, 0, 0)


def test_map_source_vector_path_and_compile():
    """exp(x0 - x1), x1 broadcast per row: 16-byte loads for x0, one scalar load for x1; 67 MB of operands
    are streamed (non-temporal), a small map of the same expression is not."""
    x0 = desc([8192, 1024])
    x1 = desc([8192, 1024], [1, 0])
    rc, src, dt = source([UN("exp"), BIN("sub"), INP(0), INP(1)], [x0, x1], desc([8192, 1024]))
    assert rc == abi.OK and dt == abi.FLOAT
    assert "const sg_float4 v0 = __builtin_nontemporal_load(" in src and "const float s1" in src and "expf((x0 - x1))" in src
    assert "__builtin_nontemporal_store(r," in src
    compiles(src)
    rc, small, _ = source([UN("exp"), BIN("sub"), INP(0), INP(1)], [desc([64, 1024]), desc([64, 1024], [1, 0])], desc([64, 1024]))
    assert rc == abi.OK and "const sg_float4 v0 = *(" in small and "nontemporal" not in small.split("extern")[1]
    compiles(small)


def test_map_source_scalar_path_for_transposed_operand():
    xt = desc([6, 4], [1, 6])
    rc, src, _ = source([UN("sin"), INP(0)], [xt], desc([6, 4]))
    assert rc == abi.OK and "float4" not in src.split("extern")[1] and "sinf(x0)" in src
    compiles(src)


def test_map_source_collapses_dense_axes():
    rc, src, _ = source([BIN("add"), INP(0), INP(1)], [desc([4, 8, 16, 32]), desc([4, 8, 16, 32])], desc([4, 8, 16, 32]))
    assert rc == abi.OK and "#define ND 1" in src
    bias = desc([32, 128, 768], [0, 0, 1])
    rc, src, _ = source([BIN("add"), INP(0), INP(1)], [desc([32, 128, 768]), bias], desc([32, 128, 768]))
    assert rc == abi.OK and "#define ND 2" in src and "const sg_float4 v1" in src


def test_every_map_operator_compiles_for_gfx950():
    """One kernel holding all 27 unary operators and one holding the binary ones + cond."""
    items = []
    for name in abi.UNARY:
        if name in ("not",):
            continue
        items = [UN(name)] + (items or [INP(0)])
    items = [UN("cast_float"), UN("not")] + items
    rc, src, dt = source(items, [desc([64, 64])], desc([64, 64]))
    assert rc == abi.OK and dt == abi.FLOAT, src
    compiles(src)
    e = [INP(0)]
    for name in ("add", "sub", "div", "mul", "pow", "min", "max"):
        e = [BIN(name)] + e + [INP(1)]
    cmp_ = lambda n: [BIN(n), INP(0), INP(1)]
    c = [BIN("and")] + cmp_("gt") + [BIN("or")] + cmp_("le") + [BIN("ne")] + cmp_("eq") + cmp_("ge")
    rc, src, dt = source([COND] + c + e + [LITF(1.5)], [desc([10, 7]), desc([10, 7])], desc([10, 7]))
    assert rc == abi.OK and dt == abi.FLOAT, src
    compiles(src)


def test_map_dtype_rules_and_errors():
    """map.rs:464-470, 491-501, 869-870; mod has no kernel (map.rs:275)."""
    f, i, u = desc([4, 4]), desc([4, 4], dtype=abi.INT), desc([4, 4], dtype=abi.UINT)
    assert source([BIN("gt"), INP(0), INP(1)], [f, f], u)[2] == abi.UINT
    assert source([UN("cast_int"), INP(0)], [f], i)[2] == abi.INT
    assert source([UN("abs"), INP(0)], [i], i)[2] == abi.INT
    assert source([UN("exp"), INP(0)], [i], f)[2] == abi.FLOAT
    assert source([UN("not"), INP(0)], [f], u)[2] == abi.UINT
    assert source([BIN("add"), INP(0), INP(1)], [f, i], f)[0] == abi.ERR_DTYPE
    assert source([COND, INP(0), INP(1), INP(1)], [f, f], f)[0] == abi.ERR_DTYPE
    assert source([BIN("gt"), INP(0), INP(1)], [f, f], f)[0] == abi.ERR_DTYPE  # output must be uint
    assert source([BIN("mod"), INP(0), INP(1)], [f, f], f)[0] == abi.ERR_ARG
    assert source([BIN("add"), INP(0)], [f], f)[0] == abi.ERR_ARG                # program ends early
    assert source([UN("exp"), INP(0)], [desc([4, 5])], f)[0] == abi.ERR_SHAPE    # ops.rs:174
    assert source([UN("exp"), INP(0)], [f], desc([4, 4], [1, 4]))[0] == abi.ERR_SHAPE  # output not dense
    assert source([UN("exp"), INP(0)], [desc([4, 4], dtype=abi.LONG)], f)[0] == abi.ERR_DTYPE


def test_gradient_graph_construction():
    """grad (var.rs:56-103) only builds graphs: no device is needed to check its structure."""
    from sage_amd import nn
    from sage_amd.grad import grad, grad_param, t_order
    from sage_amd.resnet import ResNet, ResNetConfig
    from sage_amd.tensor import UINT
    from sage_amd.var import Var
    x = Var.empty([3, 4])
    y = (x.exp() * x).sum([1], False)
    assert t_order(x) == 0 and t_order(y) == 3  # exp -> mul -> reduce (ops.rs:262-310)
    (gx,) = grad(y, [x])
    assert gx.extents == [3, 4] and gx.op == "binary" and gx.attrs["name"] == "add"  # two consumers of x: summed
    with pytest.raises(KeyError):
        grad(y, [Var.empty([2])])
    model = ResNet(ResNetConfig.d18(1, 10))
    img, lab = Var.empty([4, 28, 28, 1]), Var.empty([4, 1], UINT)
    loss = nn.softmax_cross_entropy(model.pass_(img), lab).mean(0, False)
    g = grad_param(loss, model)
    assert len(g) == 42 and all(gv.extents == p.extents for p, gv in g.items())
    ops = set()
    stack, seen = list(g.values()), set()
    while stack:
        v = stack.pop()
        if id(v) in seen:
            continue
        seen.add(id(v))
        ops.add(v.op)
        stack.extend(v.inputs)
    assert "col2im" in ops and "gemm" in ops and "cond" in ops  # conv backward, dense backward, max-pool backward


def test_model_families_build_without_a_device():
    """densenet.rs, mobilenet.rs, resnet.rs (bottleneck variants): layer trees and output shapes."""
    from sage_amd.densenet import DenseNet, DenseNetConfig
    from sage_amd.layers import fan_in_out, kaiming_normal, kaiming_uniform
    from sage_amd.mobilenet import MobileNetV2, MobileNetV2Config, make_divisible
    from sage_amd.resnet import ResNet, ResNetConfig
    from sage_amd.var import Var
    assert [make_divisible(v, 8, 8) for v in (32, 16, 24, 1280, 3, 100)] == [32, 16, 24, 1280, 8, 104]  # mobilenet.rs:10-18
    x = Var.empty([2, 32, 32, 3])
    for model, nparams in ((DenseNet(DenseNetConfig.d121(3, 10)), 236), (MobileNetV2(MobileNetV2Config(3, 10)), 106),
                           (ResNet(ResNetConfig.d50(3, 10)), 108), (ResNet(ResNetConfig.d18(3, 10)), 42)):
        assert model.pass_(x).extents == [2, 10]
        assert len(model.params()) == nparams
    # tensor/init.rs:27-50: fan_in = extents[1] * prod(extents[2:])
    assert fan_in_out([3, 3, 16, 32]) == (3 * 16 * 32, 3 * 16 * 32)
    rng = np.random.default_rng(0)
    w = kaiming_uniform(rng, [64, 256])
    assert w.dtype == np.float32 and np.abs(w).max() <= np.sqrt(3.0 / 256) + 1e-7
    assert abs(float(kaiming_normal(rng, [3, 3, 64, 64]).std()) - np.sqrt(1.0 / (3 * 64 * 64))) < 2e-3


def test_unseeded_random_nodes_are_never_merged():
    """Two unseeded fills are two independent draws (rand.rs:70, 113); seeded ones with the same seed and
    extents are the same values and may share a node."""
    from sage_amd import var as V
    a, b = V.uniform([8]), V.uniform([8])
    y = a + b
    V._merge_common_subgraphs([y])
    assert y.inputs[0] is not y.inputs[1]
    c, d = V.normal([8], (1, 2)), V.normal([8], (1, 2))
    z = c + d
    V._merge_common_subgraphs([z])
    assert z.inputs[0] is z.inputs[1]


# ------------------------------------------------------------------ state partition of Program::compile
class _DryLib:
    """Stands in for the C-ABI library on a machine without a GPU: allocations hand out fake addresses,
    every other entry point reports success.  Only the evaluator's decisions are observed, no values."""

    def __init__(self):
        self.next = 0x10000

    def sg_alloc(self, handle, nbytes, pref):
        pref._obj.value = self.next
        self.next += (int(nbytes) + 255) // 256 * 256
        return 0

    def __getattr__(self, name):
        return lambda *a: 0


class _DryCtx:
    def __init__(self):
        self._lib, self.handle, self.launches = _DryLib(), 1, 0

    def check(self, rc):
        assert rc == 0


def _data(ctx, *shape):
    import sage_amd as S
    return S.Var.new(S.Tensor.from_numpy(ctx, np.zeros(shape, np.float32)))


def test_state_partition_follows_program_compile():
    """Phase 1 of Program::compile (session.rs:101-169), worked by hand on four small graphs: candidates are the
    operator nodes with two or more consumers plus the outputs; a candidate is a state if it is an output, if a
    Contract / Reduce / Other operator lies between it and its leaves (data and earlier states), or if
    (visited nodes, leaves included) x (distinct leaves) > 5.  The evaluator must store exactly the shared map
    nodes that are states and recompute the others inside each consumer."""
    from sage_amd import nn
    from sage_amd import var as V
    ctx = _DryCtx()

    def run(targets):
        ev = V._Evaluator(ctx, targets)
        for t in targets:
            ev.get(t)
        return ev

    # 1. softmax cross-entropy as nn.rs:58-82 composes it.  c = max(x) has two consumers (x - c and log(..) + c)
    #    and is a reduce: state.  Nothing else is shared.  States: c and the output.
    x, lab = _data(ctx, 6, 10), V.Var.new(__import__("sage_amd").Tensor.from_numpy(ctx, np.zeros((6, 1), np.uint32)))
    V.set_fusion(True)
    c = x.max([1], True)
    lse = (x - c).exp().sum([1], True).log() + c
    loss = -((x - lse).gather(lab, 1).sum(1, False))
    st = V.state_partition([loss])
    assert set(st) == {id(c), id(loss)}
    assert st[id(c)] == {id(x)}                      # walk: c, x -> 2 nodes x 1 leaf, but a Reduce lies on the way
    assert st[id(loss)] == {id(x), id(c), id(lab)}   # the output's routine reads the data and the earlier state

    # 2. layer_norm as nn.rs:84-100 composes it.  mean(x) is built twice (reduce.rs:73-82); identical subgraphs are
    #    evaluated once here, so the merged mean = sum(x) / n has two consumers (x - mean and mean^2): a map node
    #    with a Reduce in its ancestry -> state, stored once rather than re-divided in both consumers.
    x = _data(ctx, 8, 16)
    g, b = _data(ctx, 1), _data(ctx, 1)
    y = nn.layer_norm_composed(x, [1], g, b, 1e-5)
    ev = run([y])
    shared_maps = [v for v in ev.keep.values() if v.op in V.MAP_OPS and ev.n_users(v) >= 2]
    mean_nodes = [v for v in shared_maps if v.op == "binary" and v.attrs["name"] == "div" and v.inputs[0].op == "reduce"]
    assert len(mean_nodes) == 1 and id(mean_nodes[0]) in ev.states and id(mean_nodes[0]) in ev.computed

    # 3. Dense + residual: h = x.W + b feeds a second Dense and the residual addition.  h is a map (the bias
    #    addition) over a Contract: state.  out = h.W2 + h is the output.
    x, w, bias, w2 = _data(ctx, 32, 16), _data(ctx, 16, 16), _data(ctx, 16), _data(ctx, 16, 16)
    h = x.matmul(w) + bias
    out = h.matmul(w2) + h
    st = V.state_partition([out])
    assert set(st) == {id(h), id(out)}
    assert st[id(out)] == {id(h), id(w2)}
    ev = run([out])
    assert id(h) in ev.computed

    # 4. shared maps without any complex operator: the threshold decides.
    #    u = -(exp(a + b)): walk u, exp, add, a, b = 5 nodes x 2 leaves = 10 > 5 -> state, stored once.
    #    w = -a: walk w, a = 2 nodes x 1 leaf = 2 -> no state, recomputed inside both consumers.
    #    s = a - b: walk s, a, b = 3 x 2 = 6 > 5 -> state.   q = a * a: walk q, a, a = 3 x 1 = 3 -> no state.
    #    (no two of these expressions share an identical sub-expression, which would be evaluated once and change the counts)
    a, b2 = _data(ctx, 4, 8), _data(ctx, 4, 8)
    u = -((a + b2).exp())
    w_ = -a
    s_ = a - b2
    q = a * a
    outs = [u * a, u + b2, w_ * b2, w_ + b2, s_.exp(), s_.log(), q.exp(), q + b2]
    st = V.state_partition(outs)
    assert id(u) in st and id(s_) in st and id(w_) not in st and id(q) not in st
    assert st[id(u)] == {id(a), id(b2)}
    ev = run(outs)
    assert id(u) in ev.computed and id(s_) in ev.computed          # materialised once
    assert id(w_) not in ev.computed and id(q) not in ev.computed  # fused into each consumer


def test_relu_factor_is_read_from_the_output_outside_relu(monkeypatch):
    """relu(h) = float(h > 0) * h (nn.rs:33-40); the backward pass multiplies by the same factor (map.rs:1014-1041).
    Before evaluation every use of the factor outside relu itself is re-pointed at float(relu(h) > 0), which has the
    same value for every h, so that h = x.W + b has one consumer and becomes the product's epilogue: one map launch
    less, and the pre-activation is never stored."""
    from sage_amd import nn
    from sage_amd import var as V
    from sage_amd.grad import grad

    class Lib(_DryLib):
        def __init__(self):
            super().__init__()
            self.log = []

        def __getattr__(self, name):
            def call(*a):
                self.log.append(name)
                return 0
            return call

    def build_and_run(ctx):
        x, w, b = _data(ctx, 8, 16), _data(ctx, 16, 32), _data(ctx, 32)
        h = x.matmul(w) + b
        y = nn.relu(h)
        loss = (y * y).sum([0, 1], False)
        gw, gb = grad(loss, [w, b])
        targets = [gw, gb, loss]
        ev = V._Evaluator(ctx, targets)
        for t in targets:
            ev.get(t)
        return h, y, ev

    V.set_fusion(True)
    ctx = _DryCtx()
    ctx._lib = Lib()
    h, y, ev = build_and_run(ctx)
    mask = next(i for i in y.inputs if i is not h)
    assert V._is_relu_mask(mask) is h
    others = [v for v in ev.keep.values() if v is not y and any(i is mask for i in v.inputs)]
    assert not others                                   # nothing but relu reads float(h > 0) any more
    assert [u for u in ev.users[id(h)] if u.op != "binary" or u.attrs["name"] not in ("gt", "mul")] == []
    assert id(h) not in ev.computed                     # folded into the product, never stored on its own
    with_rewrite = ctx._lib.log.count("sg_map")

    monkeypatch.setattr(V, "_relu_masks_from_outputs", lambda targets: None)
    ctx2 = _DryCtx()
    ctx2._lib = Lib()
    h2, _, ev2 = build_and_run(ctx2)
    assert id(h2) in ev2.computed                       # the reference's graph stores the pre-activation
    assert ctx2._lib.log.count("sg_map") == with_rewrite + 1
    assert ctx2._lib.log.count("sg_gemm") + ctx2._lib.log.count("sg_matmul_strided") == ctx._lib.log.count("sg_gemm") + ctx._lib.log.count("sg_matmul_strided")


def test_pool_model_keeps_an_allocators_invariants():
    """The host-side model the GPU tests hold the chunked allocator against (tests/pool_model.py), on its own: blocks
    handed out never overlap, every byte of every chunk is in exactly one block (handed out or free), free neighbours
    never stay apart, the figures add up, and the capacity bounds the chunks held."""
    import numpy as np
    from tests import pool_model as PM
    for seed, capacity, sub in [(0, 0, True), (1, 128 * PM.MIB, True), (2, 64 * PM.MIB, True), (3, 128 * PM.MIB, False)]:
        rng = np.random.default_rng(seed)
        m = PM.Pool(capacity, sub)
        live = []
        for step in range(1500):
            if live and (rng.random() < 0.48 or len(live) > 60):
                m.free(live.pop(int(rng.integers(len(live)))))
            else:
                r = rng.random()
                n = int(rng.integers(1, 1 << 16)) if r < 0.4 else int(rng.integers(1 << 16, 3 << 20)) if r < 0.8 else int(rng.integers(3 << 20, 30 << 20))
                try:
                    chunk, off, size = m.alloc(n)
                except PM.OutOfMemory:
                    assert capacity, "an unbounded pool cannot run out"
                    continue
                assert size >= n and off % PM.ALIGN == 0
                live.append((chunk, off))
            blocks = [(b.chunk, b.offset, b.size, b.cap, "live") for b in m.live.values()]
            blocks += [(b.chunk, b.offset, b.size, b.cap, "free") for b in m.small + m.large]
            by_chunk = {}
            for c, o, s, cap, kind in blocks:
                by_chunk.setdefault(c, []).append((o, s, cap, kind))
            total = 0
            for c, parts in by_chunk.items():
                parts.sort()
                assert parts[0][0] == 0 and all(a[0] + a[1] == b[0] for a, b in zip(parts, parts[1:])), f"step {step}: chunk {c} has a hole or an overlap"
                assert parts[-1][0] + parts[-1][1] == parts[0][2]
                if sub:
                    assert not any(a[3] == b[3] == "free" for a, b in zip(parts, parts[1:])), f"step {step}: free neighbours left apart"
                total += parts[0][2]
            assert total == m.total and m.used == sum(b.size for b in m.live.values()) and m.peak >= m.total
            assert not capacity or m.total <= capacity
        for k in live:
            m.free(k)
        m.trim()
        assert m.used == 0 and m.total == 0 and not m.small and not m.large
