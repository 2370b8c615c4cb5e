#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X: BERT-base forward (b32, s128, fp32) through the C ABI.

A step is one full forward pass (embedding gathers + LayerNorm, 12 encoder layers, classifier) over
one synthetic batch that is already resident in HBM.  The model is the configuration the metric is
quoted on — erf-GELU, LayerNorm eps 1e-12 with per-feature gamma/beta, weights ~N(0, 0.02) — built
from the same operators the parity tests check; `--variant reference` runs the composition the
reference's own models/bert.rs builds instead (ReLU, eps 1e-5, scalar gamma = beta).

Prints ONE JSON line: whole-job throughput, the roofline of the dominant kernel (the fp32 MFMA
GEMM instantiation that takes the most time, timed per launch with HIP events on the stream it
runs on, inside the timed steps) and the CPU oracle timed on a bounded sample of the same workload.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0
# `traffic` is not measured by this run: it is read, by kernel name, from the committed counter summaries under profiles/
# (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this same workload); it goes stale if the kernel changes and they are not re-collected
TRAFFIC_SOURCE = "profiles/traffic_*.json (committed rocprofv3 --pmc summary of this workload, looked up by kernel name; not measured in this run)"


def measured_traffic(kernel, workload):
    """HBM bytes per dispatch of `kernel` from the committed rocprofv3 counter summary of this same
    workload (FETCH_SIZE and WRITE_SIZE runs scaled by a copy kernel of known size), or None when there
    is no such measurement.  profiles/traffic_<workload>.json holds every kernel of a model workload;
    profiles/traffic_single_kernel_workloads.json holds the one timed kernel of each single-kernel workload."""
    try:
        with open(os.path.join(ROOT, "profiles", f"traffic_{workload}.json")) as f:
            k = json.load(f)["kernels"].get(kernel)
        return k["traffic_bytes_per_dispatch"] if k else None
    except (OSError, ValueError, KeyError):
        pass
    try:
        with open(os.path.join(ROOT, "profiles", "traffic_single_kernel_workloads.json")) as f:
            return json.load(f)["workloads"][workload]["traffic_bytes_per_dispatch"]
    except (OSError, ValueError, KeyError):
        return None


def build_bert(ctx, variant, batch, seq, layers, rng, detail=False):
    """The model the metric is quoted on.  variant "config": erf-GELU, LayerNorm eps 1e-12 with per-feature
    gamma/beta, a 2-row segment table with segment ids, classifier on token 0.  variant "reference": what the
    reference's models/bert.rs composes (ReLU, eps 1e-5, scalar gamma = beta = 1, no segment table, token 1).
    detail=True also returns the host arrays (params() order), inputs and the last encoder output, for the
    parity tests that rebuild the same model on the CPU."""
    import sage_amd as S
    from sage_amd.bert import Bert, BertConfig
    cfg = BertConfig.base()
    cfg.num_layers = layers
    exact = variant == "reference"
    model = Bert(cfg, reference_exact=exact, segments=0 if exact else 2)
    arrays = []
    for p in model.params():
        n = p.label or ""
        if "layer_norm.gamma" in n:
            a = np.ones(p.extents, np.float32)
        elif "layer_norm.beta" in n:
            a = np.ones(p.extents, np.float32) if exact else np.zeros(p.extents, np.float32)
        elif n.endswith(".bias"):
            a = np.zeros(p.extents, np.float32)
        else:
            a = (rng.standard_normal(p.extents) * 0.02).astype(np.float32)
        arrays.append(a)
        p.set(S.Tensor.from_numpy(ctx, a))
    ids = rng.integers(0, cfg.num_vocabs, (batch, seq)).astype(np.int32)
    mask = np.ones((batch, seq), np.float32)
    seg = None if exact else rng.integers(0, 2, (batch, seq)).astype(np.int32)
    ids_v = S.Var.new(S.Tensor.from_numpy(ctx, ids))
    mask_v = S.Var.new(S.Tensor.from_numpy(ctx, mask))
    seg_v = None if seg is None else S.Var.new(S.Tensor.from_numpy(ctx, seg))
    hidden = model.encode(model.embedding.pass_(ids_v, ctx, seg_v), mask_v)
    logits = model.classify(hidden)
    if detail:
        return {"cfg": cfg, "model": model, "logits": logits, "hidden": hidden, "arrays": arrays, "ids": ids, "mask": mask, "segment_ids": seg}
    return cfg, model, logits


def build_resnet18(ctx, batch, rng):
    """ResNet-18 on [batch, 28, 28, 1] images (the reference's MNIST example shape), Kaiming-normal filters."""
    import sage_amd as S
    from sage_amd.resnet import ResNet, ResNetConfig
    model = ResNet(ResNetConfig.d18(1, 10))
    arrays = []
    for p in model.params():
        ext = p.extents
        if len(ext) == 1:
            a = np.zeros(ext, np.float32)
        elif len(ext) == 4:
            a = (rng.standard_normal(ext) * np.sqrt(2.0 / (ext[0] * ext[1] * ext[2]))).astype(np.float32)
        else:
            a = (rng.standard_normal(ext) * 0.05).astype(np.float32)
        arrays.append(a)
        p.set(S.Tensor.from_numpy(ctx, a))
    x = rng.uniform(0, 1, (batch, 28, 28, 1)).astype(np.float32)
    return model, arrays, x, model.pass_(S.Var.new(S.Tensor.from_numpy(ctx, x)))


def cpu_baseline_resnet18(model, arrays, x):
    """The CPU oracle on the whole ResNet-18 forward pass at the bench's batch."""
    from oracle import oracle as O
    ht = O.HT.from_numpy
    it = iter(arrays)
    pod = {"w0": ht(next(it)), "b0": ht(next(it)), "blocks": []}
    inp, out = 64, 64
    for i in range(4):
        ip = inp
        for b in range(2):
            s = (1 if i == 0 else 2) if b == 0 else 1
            blk = {"stride": s, "w1": ht(next(it)), "b1": ht(next(it)), "w2": ht(next(it)), "b2": ht(next(it))}
            if s != 1 or ip != out:
                blk["wd"], blk["bd"] = ht(next(it)), ht(next(it))
            pod["blocks"].append(blk)
            ip = out
        inp, out = out, out * 2
    pod["wfc"], pod["bfc"] = ht(next(it)), ht(next(it))
    t0 = time.perf_counter()
    O.resnet18_forward(ht(x), pod)
    dt = time.perf_counter() - t0
    return {"value": x.shape[0] / dt, "unit": "images/s", "cores": O.num_threads(), "kind": "port",
            "sample": f"one whole forward pass at b{x.shape[0]} in {dt:.2f} s"}


def gemm_calls(ctx, prog):
    """(call index, kernel name, flops, shape) for every GEMM launch of the compiled program.  The name is what
    the library reports right after the call has been issued once more (tile, layouts, guarded loads and image
    addressing are template arguments chosen per shape)."""
    from sage_amd import abi
    lib = abi.lib()
    out = []

    def launched(fn, args):
        ctx.check(fn(ctx.handle, *args))
        buf = C.create_string_buffer(128)
        ctx.check(lib.sg_gemm_last_kernel_name(ctx.handle, buf, 128))
        return buf.value.decode()
    for i, (fn, args, _) in enumerate(prog.calls):
        if fn is lib.sg_conv2d:  # the product of the never-written column matrix [N*OH*OW, KH*KW*C] with the filter [KH*KW*C, OC]
            x, f, c = (a._obj for a in args[:3])
            M, N, K = c.extents[0] * c.extents[1] * c.extents[2], c.extents[3], f.extents[0] * f.extents[1] * f.extents[2]
            out.append((i, launched(fn, args), 2.0 * M * N * K + M * N, (M, N, K, 1)))
            continue
        if fn in (lib.sg_gemm, lib.sg_gemm_batched, lib.sg_matmul_strided):
            if fn is lib.sg_matmul_strided:
                a, b, c = (x._obj for x in args[:3])
                ta = 0
            else:
                ta = args[0]
                a, b, c = (x._obj for x in args[2:5])
            r = c.rank
            M, N = c.extents[r - 2], c.extents[r - 1]
            K = a.extents[r - 1] if fn is lib.sg_matmul_strided or not ta else a.extents[r - 2]
            batch = 1
            for d in range(r - 2):
                batch *= c.extents[d]
            out.append((i, launched(fn, args), 2.0 * M * N * K * batch + M * N * batch, (M, N, K, batch)))
    return out


def run_timed(ctx, prog, timed):
    """One replay of the program with a HIP event pair around each call index in `timed`."""
    from sage_amd import abi
    lib = abi.lib()
    h = ctx.handle
    for i, (fn, args, _) in enumerate(prog.calls):
        if i in timed:
            a, b = timed[i]
            lib.sg_event_record(h, a)
            rc = fn(h, *args)
            lib.sg_event_record(h, b)
        else:
            rc = fn(h, *args)
        if rc:
            ctx.check(rc)


def opencl_cpu_devices():
    """How many CPU devices the installed OpenCL platforms offer (the reference runs on whatever OpenCL device it
    finds, session/device.rs:36-70; a CPU OpenCL device, e.g. PoCL, would run its own kernels on the host cores).
    Returns (count, description); (0, why) when there is no loader, no platform or no CPU device."""
    try:
        cl = C.CDLL("libOpenCL.so.1")
    except OSError:
        return 0, "no OpenCL loader"
    n = C.c_uint(0)
    if cl.clGetPlatformIDs(0, None, C.byref(n)) != 0 or n.value == 0:
        return 0, "OpenCL loader present, no platform"
    plats = (C.c_void_p * n.value)()
    cl.clGetPlatformIDs(n.value, plats, None)
    CL_DEVICE_TYPE_CPU, CL_PLATFORM_NAME = C.c_ulong(1 << 1), 0x0902
    total, names = 0, []
    for p in plats:
        buf = C.create_string_buffer(256)
        cl.clGetPlatformInfo(C.c_void_p(p), CL_PLATFORM_NAME, 256, buf, None)
        nd = C.c_uint(0)
        rc = cl.clGetDeviceIDs(C.c_void_p(p), CL_DEVICE_TYPE_CPU, 0, None, C.byref(nd))
        names.append(f"{buf.value.decode(errors='replace')}: {nd.value if rc == 0 else 0} CPU devices")
        total += nd.value if rc == 0 else 0
    return total, "; ".join(names)


def cpu_baseline_kind(entry):
    """The CPU leg is the oracle (a C port of the reference's kernels).  The reference itself needs a Rust nightly
    toolchain to build and an OpenCL device to run; the probe records whether the box would at least have offered
    a CPU OpenCL device to it."""
    n, what = opencl_cpu_devices()
    entry["opencl_cpu_devices"] = n
    entry["opencl_probe"] = what
    return entry


LAYER_KEYS = ["wk", "bk", "wq", "bq", "wv", "bv", "wo", "bo", "ln1_g", "ln1_b", "w1", "b1", "w2", "b2", "ln2_g", "ln2_b"]


def cpu_baseline_whole_model(bert, variant, layers, gpu_logits):
    """The CPU oracle on the whole model the GPU leg timed: same weights, same token ids, embedding to
    classifier (about 10 s at b32 x s128 on 16 threads).  The worst deviation of the GPU logits from the
    oracle's is reported beside the rate."""
    from oracle import oracle as O
    ht = O.HT.from_numpy
    it = iter(bert["arrays"])
    exact = variant == "reference"
    p = {"word_emb": ht(next(it)), "pos_emb": ht(next(it))}
    if not exact:
        p["seg_emb"] = ht(next(it))
    p["emb_g"], p["emb_b"] = ht(next(it)), ht(next(it))
    p["layers"] = [{k: ht(next(it)) for k in LAYER_KEYS} for _ in range(layers)]
    p["wc"], p["bc"] = ht(next(it)), ht(next(it))
    act, eps, cls = ("relu", 1e-5, 1) if exact else ("gelu", 1e-12, 0)
    ids, seg = ht(bert["ids"].view(np.uint32)), None if bert["segment_ids"] is None else ht(bert["segment_ids"].view(np.uint32))
    batch, seq = bert["ids"].shape
    t0 = time.perf_counter()
    lo = O.bert_forward(ids, ht(bert["mask"]), p, 12, act, eps, cls, seg)
    dt = time.perf_counter() - t0
    lo = lo.numpy().astype(np.float64)
    dev = float(np.max(np.abs(gpu_logits - lo) / np.maximum(np.abs(lo), np.sqrt(np.mean(lo * lo)))))
    return cpu_baseline_kind({"value": batch / dt, "unit": "seqs/s", "cores": O.num_threads(), "kind": "port",
                              "sample": f"the whole {layers}-layer forward pass at b{batch} s{seq} (same weights and ids) in {dt:.1f} s",
                              "gpu_vs_cpu_logits_worst_rel": dev})


def cpu_baseline(variant, batch, seq, rng_seed):
    """The CPU oracle (oracle/: C restatement of the reference kernels, OpenMP over work-items) on one
    of the 12 encoder layers (whole batch at b32 x s128; at most 4096 tokens of it for larger shapes);
    the layer time x 12 gives seqs/s."""
    from oracle import oracle as O
    rng = np.random.default_rng(rng_seed)
    e, hdim, heads = 768, 3072, 12
    w = lambda i, o: O.HT.from_numpy((rng.standard_normal((i, o)) * 0.02).astype(np.float32))
    z = lambda n: O.HT.from_numpy(np.zeros(n, np.float32))
    nln = 1 if variant == "reference" else e
    one = lambda: O.HT.from_numpy(np.ones(nln, np.float32))
    p = {"wq": w(e, e), "bq": z(e), "wk": w(e, e), "bk": z(e), "wv": w(e, e), "bv": z(e), "wo": w(e, e), "bo": z(e),
         "ln1_g": one(), "ln1_b": z(nln), "w1": w(e, hdim), "b1": z(hdim), "w2": w(hdim, e), "b2": z(e), "ln2_g": one(), "ln2_b": z(nln)}
    batch = max(1, min(batch, 4096 // seq))  # bounded sample: at most 4096 tokens
    x = O.HT.from_numpy(rng.standard_normal((batch, seq, e)).astype(np.float32))
    mask = O.HT.from_numpy(np.ones((batch, seq), np.float32))
    act, eps = ("relu", 1e-5) if variant == "reference" else ("gelu", 1e-12)
    t0 = time.perf_counter()
    O.bert_layer(x, mask, p, heads, act, eps)
    dt = time.perf_counter() - t0
    return cpu_baseline_kind({"value": batch / (12.0 * dt), "unit": "seqs/s", "cores": O.num_threads(), "kind": "port",
                              "sample": f"1 of 12 encoder layers at b{batch} s{seq} in {dt:.2f} s, x12 (embedding and classifier left out)"})


# --------------------------------------------------------------------------------------------
# Single-kernel workloads (the other configurations the parity tests cover).  Each rotates over
# enough distinct buffer sets to exceed the 256 MB Infinity Cache, so the rate is an HBM rate.
def kernel_workloads(ctx, name, rng, elements=None):
    """name -> (list of programs to rotate over, algorithmic bytes per call, flops per call,
    kernel label, spec of the oracle's CPU baseline or None).  Every buffer set is a distinct device
    allocation (so the caches cannot serve the next launch) filled from one host array."""
    import sage_amd as S
    from sage_amd import nn

    def dev(a):
        return S.Var.new(S.Tensor.from_numpy(ctx, a))

    def programs(build, nbuf):
        return [S.Program(ctx, [build(i)]) for i in range(nbuf)]

    def normal(*shape):
        return rng.standard_normal(shape, dtype=np.float32)

    if name == "softmax_ce":      # config 1: logits [8192,1024] f32, labels int32 -> loss [8192]
        B, Cn = 8192, 1024
        lab, x = rng.integers(0, Cn, (B, 1)).astype(np.int32), normal(B, Cn)
        progs = programs(lambda i: nn.softmax_cross_entropy(dev(x), dev(lab)), 20)
        return progs, B * Cn * 4 + B * 4 + B * 4, 0.0, "softmax_ce_row_kernel<4, 64>", ("softmax_ce", B, Cn)
    if name == "map_exp_sub":     # exp(x0 - x1), x1 broadcast per row (the largest map of config 1)
        B, Cn = 8192, 1024
        c, x = normal(B, 1), normal(B, Cn)
        progs = programs(lambda i: (dev(x) - dev(c)).exp(), 12)
        return progs, 2 * B * Cn * 4 + B * 4, 0.0, "sg_map", ("map_exp_sub", B, Cn)
    if name == "bias_residual":   # (g + bias) + x on [4096, 3072]: 3-input fused map
        M, N = 4096, 3072
        bias, g, x = normal(N), normal(M, N), normal(M, N)
        progs = programs(lambda i: (dev(g) + dev(bias)) + dev(x), 8)
        return progs, 3 * M * N * 4 + N * 4, 0.0, "sg_map", None
    if name == "layer_norm":      # [32768, 768] rows (BERT b64 s512), per-feature gamma/beta
        R, Cn = 32768, 768
        g, b, x = dev(np.ones(Cn, np.float32)), dev(np.zeros(Cn, np.float32)), normal(R, Cn)
        progs = programs(lambda i: nn.layer_norm(dev(x), 1, g, b, 1e-12), 6)
        return progs, 2 * R * Cn * 4 + 2 * Cn * 4, 0.0, "layer_norm_row_kernel<3, 64, true>", None
    if name == "softmax":         # attention scores [32,12,128,128] + mask
        n, h, l = 32, 12, 128
        m, x = dev(np.zeros((n, 1, 1, l), np.float32)), normal(n, h, l, l)
        progs = programs(lambda i: nn.softmax(dev(x) + m, 3), 12)
        return progs, 2 * n * h * l * l * 4 + n * l * 4, 0.0, "softmax_row_kernel<4, 8, true, true>", None
    if name == "reduce_sum":      # row sums of [8192,1024]
        B, Cn = 8192, 1024
        x = normal(B, Cn)
        progs = programs(lambda i: dev(x).sum(1, True), 20)
        return progs, B * Cn * 4 + B * 4, 0.0, "reduce_row_kernel<0, float, true, false>", None
    if name == "copy":            # plain copy (64 Mi floats by default): the kernel of known size that calibrates FETCH_SIZE / WRITE_SIZE;
        n = int(elements) if elements else 64 << 20   # with --elements, the copy that moves as many bytes as another workload (its ceiling)
        x = np.ones(n, np.float32)
        nbuf = max(1, min(24, (600 << 20) // (8 * n)))  # enough buffer sets to exceed the 256 MB Infinity Cache
        progs = programs(lambda i: dev(x).copy(), nbuf)
        return progs, 2 * n * 4, 0.0, "sg_map", None
    if name == "launch_floor":    # a copy of 1024 floats: what one launch costs in a back-to-back stream when it moves nothing
        progs = programs(lambda i: dev(np.ones(1024, np.float32)).copy(), 4)
        return progs, 2 * 1024 * 4, 0.0, "sg_map", None
    if name == "gemm_bias":       # config 2: C = A@B + bias, 4096^3
        M = N = K = 4096
        A, Bm, bias = (dev(rng.uniform(-1, 1, s).astype(np.float32)) for s in ((M, K), (K, N), (N,)))
        progs = programs(lambda i: A.matmul(Bm) + bias, 2)
        return progs, 4.0 * (M * K + K * N + M * N + N), 2.0 * M * N * K + M * N, "gemm_mfma_kernel<128, 128, 2, true, true, false, false, true>", ("gemm", M, N, K)
    raise SystemExit(f"unknown workload {name}")


def oracle_kernel_baseline(spec, rng):
    from oracle import oracle as O
    kind = spec[0]
    if kind == "softmax_ce":
        _, B, Cn = spec
        x = O.HT.from_numpy(rng.standard_normal((B, Cn)).astype(np.float32))
        lab = O.HT.from_numpy(rng.integers(0, Cn, (B, 1)).astype(np.uint32))
        t0 = time.perf_counter()
        O.softmax_cross_entropy(x, lab)
        return time.perf_counter() - t0, f"one softmax_cross_entropy of [{B},{Cn}] (8 un-fused launches)"
    if kind == "map_exp_sub":
        _, B, Cn = spec
        x = O.HT.from_numpy(rng.standard_normal((B, Cn)).astype(np.float32))
        c = O.HT.from_numpy(rng.standard_normal((B, 1)).astype(np.float32))
        E = O.E
        t0 = time.perf_counter()
        O.fused_map(E.un("exp", E.bin("sub", E.inp(0), E.inp(1))), [x, c.expand([B, Cn])], O.FLOAT)
        return time.perf_counter() - t0, f"one fused exp(x0-x1) over [{B},{Cn}]"
    if kind == "gemm":
        _, M, N, K = spec
        m = 512  # a 512-row block of A: 1/8 of the work
        a = O.HT.from_numpy(rng.uniform(-1, 1, (m, K)).astype(np.float32))
        b = O.HT.from_numpy(rng.uniform(-1, 1, (K, N)).astype(np.float32))
        bias = O.HT.from_numpy(rng.uniform(-1, 1, (N,)).astype(np.float32))
        t0 = time.perf_counter()
        O.dense(a, b, bias)
        return (time.perf_counter() - t0) * (M / m), f"a {m}-row block of A (1/{M // m} of the GEMM), scaled x{M // m}"
    return None, None


def time_kernel_workload(ctx, name, steps, warmup, elements=None):
    """Times `steps` launches of one single-kernel workload (after `warmup`) between two HIP events on the
    context's stream, rotating over its buffer sets.  Returns (roofline dict, config dict, oracle spec)."""
    from sage_amd import abi
    lib = abi.lib()
    progs, bytes_per, flops_per, label, spec = kernel_workloads(ctx, name, np.random.default_rng(1), elements)
    launches = len(progs[0].calls)

    def ev():
        e = C.c_void_p()
        ctx.check(lib.sg_event_create(ctx.handle, C.byref(e)))
        return e

    for i in range(warmup):
        progs[i % len(progs)].run()
    ctx.sync()
    e0, e1 = ev(), ev()
    t0 = time.perf_counter()
    lib.sg_event_record(ctx.handle, e0)
    for i in range(steps):
        progs[i % len(progs)].run()
    lib.sg_event_record(ctx.handle, e1)
    ctx.sync()
    wall_ms = (time.perf_counter() - t0) / steps * 1e3
    ms = C.c_float()
    ctx.check(lib.sg_event_elapsed_ms(ctx.handle, e0, e1, C.byref(ms)))
    for e in (e0, e1):
        lib.sg_event_destroy(ctx.handle, e)
    per_ms = ms.value / steps
    if flops_per:
        achieved, peak, unit, bound = flops_per / (per_ms * 1e-3) / 1e12, PEAK_FP32_MFMA_TFLOPS, "TFLOP/s", "mfma"
    else:
        achieved, peak, unit, bound = bytes_per / (per_ms * 1e-3) / 1e9, PEAK_HBM_GBS, "GB/s", "hbm"
    roof = {"bound": bound, "achieved": achieved, "peak": peak, "unit": unit, "frac": achieved / peak,
            "traffic": measured_traffic(label, name), "kernel": label, "avg_launch_ms": per_ms}
    roof["traffic_source"] = TRAFFIC_SOURCE if roof["traffic"] is not None else None
    cfg = {"workload": name, "launches_per_step": launches, "buffer_sets": len(progs),
           "algorithmic_bytes_per_step": bytes_per, "flops_per_step": flops_per, "wall_ms_per_step": wall_ms}
    del progs
    return roof, cfg, spec


# The HBM half of the metric: the fused map / reduce / row kernels at the shapes of configurations 1, 3 and 5.
HBM_WORKLOADS = ("softmax_ce", "reduce_sum", "map_exp_sub", "softmax", "bias_residual", "layer_norm")


def hbm_rooflines(ctx, steps=2000, warmup=500):
    """One roofline entry per fused HBM-bound kernel, each timed back to back on rotating buffer sets."""
    out = []
    for name in HBM_WORKLOADS:
        roof, cfg, _ = time_kernel_workload(ctx, name, steps, warmup)
        ctx.trim()
        nbytes = cfg["algorithmic_bytes_per_step"]
        # the bound that travels with the number: a plain streaming copy that moves the same number of bytes, same run
        copy, _, _ = time_kernel_workload(ctx, "copy", steps, warmup, elements=max(1024, nbytes // 8 // 4 * 4))
        ctx.trim()
        out.append({"workload": name, "kernel": roof["kernel"], "bytes": nbytes,
                    "avg_launch_ms": roof["avg_launch_ms"], "achieved": roof["achieved"], "unit": "GB/s",
                    "frac": roof["frac"], "copy_frac": copy["frac"], "copy_avg_launch_ms": copy["avg_launch_ms"],
                    "traffic": roof["traffic"], "traffic_source": TRAFFIC_SOURCE if roof["traffic"] is not None else None, "launches_timed": steps})
    return out


def run_kernel_workload(a):
    import sage_amd as S
    ctx = S.Context(0)
    roof, cfg, spec = time_kernel_workload(ctx, a.workload, a.steps, a.warmup, a.elements)
    unit, flops_per, bytes_per = roof["unit"], cfg["flops_per_step"], cfg["algorithmic_bytes_per_step"]
    res = {"metric": f"{a.workload} throughput", "value": roof["achieved"], "unit": unit, "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
           "ms_per_step": cfg.pop("wall_ms_per_step"), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
           "data": "synthetic", "config": cfg, "roofline": roof}
    if spec is not None and not a.no_cpu_baseline:
        t, sample = oracle_kernel_baseline(spec, np.random.default_rng(2))
        if t:
            from oracle import oracle as O
            v = (flops_per / t / 1e12) if flops_per else (bytes_per / t / 1e9)
            res["cpu_baseline"] = {"value": v, "unit": unit, "cores": O.num_threads(), "kind": "port", "sample": sample}
    print(json.dumps(res))


def run_train_workload(a):
    """One training step of examples/train.rs: ResNet-18 on [B,28,28,1] -> mean softmax-CE -> grad_param -> Adam,
    as two replayed programs (forward+backward, optimizer update)."""
    import sage_amd as S
    from sage_amd import nn, optim
    from sage_amd.grad import grad_param
    ctx = S.Context(0)
    rng = np.random.default_rng(4)
    batch = a.batch if a.batch != 32 else 128
    model, arrays, x_host, logits = build_resnet18(ctx, batch, rng)
    labels = rng.integers(0, 10, (batch, 1)).astype(np.int32)
    loss = nn.softmax_cross_entropy(logits, S.Var.new(S.Tensor.from_numpy(ctx, labels))).mean(0, False)
    grads = grad_param(loss, model)
    prog = S.Program(ctx, list(grads.values()) + [loss]).bind()
    opt = optim.Adam(1e-4)
    opt.init(ctx)
    opt.update(grads, ctx)           # the reference's first update only creates the (zero) moments
    upd = opt.compile(grads, ctx)
    use_graph = a.graph != "off"
    if use_graph:
        prog.capture()
        upd.capture()
    gflops = sum(f for _, _, f, _ in gemm_calls(ctx, prog))
    for _ in range(a.warmup):
        prog.run()
        upd.run()
    ctx.sync()
    loss0 = float(prog.outputs[-1].numpy()[0])
    t0 = time.perf_counter()
    for _ in range(a.steps):
        prog.run()
        upd.run()
    ctx.sync()
    dt = time.perf_counter() - t0
    loss1 = float(prog.outputs[-1].numpy()[0])
    if not (np.isfinite(loss1) and loss1 < loss0):
        raise SystemExit(f"training on a fixed batch did not reduce the loss ({loss0} -> {loss1})")
    ms = dt / a.steps * 1e3
    achieved = gflops / (ms * 1e-3) / 1e12
    res = {"metric": f"ResNet-18 train step images/sec (b{batch},28x28x1,fp32,Adam)", "value": batch / (ms * 1e-3), "unit": "images/s",
           "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": f"resnet18_train_b{batch}_28x28x1_fp32_adam", "replay": "hip_graph" if use_graph else "eager",
                      "launches_per_step": len(prog.calls) + len(upd.calls), "loss_first": loss0, "loss_last": loss1},
           "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                        "frac": achieved / PEAK_FP32_MFMA_TFLOPS, "traffic": None,
                        "kernel": "all GEMM launches of the step over the whole step time (the step is launch- and HBM-bound, no single dominant kernel)"}}
    print(json.dumps(res))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="bert", help="bert (default, the headline metric) | resnet18 | resnet18_train | copy | launch_floor | softmax_ce | map_exp_sub | "
                    "bias_residual | layer_norm | softmax | reduce_sum | gemm_bias")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default 30; 2000 for the single-kernel workloads, whose step is microseconds)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default 5; 500 for the single-kernel workloads)")
    ap.add_argument("--variant", choices=["config", "reference"], default="config")
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--seq", type=int, default=128)
    ap.add_argument("--layers", type=int, default=12)
    ap.add_argument("--elements", type=int, default=None, help="copy workload: number of floats copied (default 64 Mi)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true", help="bert at the headline shape: leave out the `configs` list (the other four configurations timed behind it)")
    ap.add_argument("--no-hbm-kernels", action="store_true", help="bert: leave out the roofline_hbm list (the fused map/reduce/row kernels timed after the model)")
    ap.add_argument("--graph", choices=["auto", "on", "off"], default="auto",
                    help="replay the step as one HIP graph (auto = on; off: one host call per operator launch)")
    a = ap.parse_args()
    single_kernel = a.workload not in ("bert", "resnet18", "resnet18_train")
    if a.steps is None:
        a.steps = 2000 if single_kernel else 30
    if a.warmup is None:
        a.warmup = 500 if single_kernel else 5
    if a.gpus != 1:
        print("bench.py measures one GPU: every box in this run has one MI355X and the hot path uses no "
              "collectives; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if a.workload == "resnet18_train":
        return run_train_workload(a)
    if a.workload not in ("bert", "resnet18"):
        return run_kernel_workload(a)

    import sage_amd as S
    ctx = S.Context(0)
    res, keep = time_model(ctx, a.workload, a.variant, a.batch, a.seq, a.layers, a.steps, a.warmup, a.graph != "off")
    headline = a.workload == "bert" and (a.batch, a.seq, a.layers, a.variant) == (32, 128, 12, "config")
    # The headline is measured; what follows adds to the line.  A failure in one of the additions is reported in the
    # line (`<key>_error`) instead of costing the headline its record.
    def added(key, make):
        try:
            res[key] = make()
        except Exception as e:  # noqa: BLE001
            res[key + "_error"] = f"{type(e).__name__}: {e}"[:400]
            print(f"bench.py: {key} failed: {e}", file=sys.stderr)

    if a.workload == "bert" and not a.no_hbm_kernels:
        # the other half of the metric: the fused map / reduce / row kernels against the HBM peak, each beside a
        # plain copy of the same number of bytes timed in this same run (what a launch of that size can reach)
        ctx.trim()
        added("roofline_hbm", lambda: hbm_rooflines(ctx))
    if headline and not a.no_configs:
        added("configs", lambda: other_configs(ctx, res))
    if not a.no_cpu_baseline:
        if a.workload == "resnet18":
            added("cpu_baseline", lambda: cpu_baseline_resnet18(keep["model"], keep["arrays"], keep["x_host"]))
        elif a.batch * a.seq <= 4096:
            added("cpu_baseline", lambda: cpu_baseline_whole_model(keep["bert"], a.variant, a.layers, keep["out0"]))
        else:
            added("cpu_baseline", lambda: cpu_baseline(a.variant, a.batch, a.seq, 6))
    print(json.dumps(res))


def time_model(ctx, workload, variant, batch, seq, layers, steps, warmup, use_graph):
    """Builds a model workload (bert | resnet18), runs `warmup` untimed and `steps` timed forward passes and times
    the launches of its dominant GEMM instantiation with HIP event pairs on the context's stream.  Returns the
    result line (metric, value, config, roofline) and what the CPU baseline needs (host arrays, first output).
    Every device buffer of the model is released before returning."""
    import sage_amd as S
    from sage_amd import abi
    lib = abi.lib()
    rng = np.random.default_rng(5)
    keep = {}
    if workload == "resnet18":
        batch = batch if batch != 32 else 128
        model, arrays, x_host, logits = build_resnet18(ctx, batch, rng)
        keep.update(model=model, arrays=arrays, x_host=x_host)
    else:
        bert = build_bert(ctx, variant, batch, seq, layers, rng, detail=True)
        cfg, model, logits = bert["cfg"], bert["model"], bert["logits"]
        keep.update(bert=bert)
    prog = S.Program(ctx, [logits])  # first evaluation: builds kernels, allocates every buffer
    ctx.sync()
    out0 = prog.outputs[0].numpy()
    keep["out0"] = out0
    if not np.all(np.isfinite(out0)):
        raise SystemExit("non-finite model output")

    # the dominant kernel: the GEMM instantiation with the most flops in the program
    gc = gemm_calls(ctx, prog)
    by_name = {}
    for i, name, flops, shape in gc:
        by_name.setdefault(name, []).append((i, flops, shape))
    dom = max(by_name, key=lambda n: sum(f for _, f, _ in by_name[n]))

    def new_event():
        e = C.c_void_p()
        ctx.check(lib.sg_event_create(ctx.handle, C.byref(e)))
        return e

    # Event pairs around launches of the dominant kernel, read after the timed region.  An event record is
    # a marker packet in the queue and costs about 3 us of stream time (72 of them made a 5.6 ms BERT step
    # 5.8 ms), so a step brackets only every SAMPLE-th launch of the kernel and the steps rotate through
    # the launches: every launch index is timed in steps/SAMPLE of the timed steps.
    SAMPLE = 6
    dom_calls = [i for i, _, _ in by_name[dom]]
    pairs = [{i: (new_event(), new_event()) for j, i in enumerate(dom_calls) if j % SAMPLE == step % SAMPLE} for step in range(max(steps, SAMPLE))]

    if use_graph:
        prog.capture()
    for _ in range(warmup):
        prog.run()
    ctx.sync()
    t0 = time.perf_counter()
    if use_graph:
        # the timed region replays the graph; the dominant kernel's launches are timed with event
        # pairs in an eager replay of the same steps right behind it (events cannot bracket graph nodes)
        for step in range(steps):
            prog.run()
        ctx.sync()
        dt = time.perf_counter() - t0
        for step in range(len(pairs)):
            run_timed(ctx, prog, pairs[step])
        ctx.sync()
    else:
        for step in range(steps):
            run_timed(ctx, prog, pairs[step])
        ctx.sync()
        dt = time.perf_counter() - t0
        for step in range(steps, len(pairs)):
            run_timed(ctx, prog, pairs[step])
        ctx.sync()
    flops_of = {i: f for i, f, _ in by_name[dom]}
    ms_of = {i: [] for i in flops_of}
    for step in range(len(pairs)):
        for i, (e0, e1) in pairs[step].items():
            ms = C.c_float()
            ctx.check(lib.sg_event_elapsed_ms(ctx.handle, e0, e1, C.byref(ms)))
            ms_of[i].append(ms.value)
            lib.sg_event_destroy(ctx.handle, e0)
            lib.sg_event_destroy(ctx.handle, e1)
    ms_per_step = dt / steps * 1e3

    # Every launch index of the kernel counts once, whatever number of steps sampled it: the mean duration of
    # each index first, then flops and time summed over the indices (all of them are sampled: at least SAMPLE replays).
    sampled = [i for i in ms_of if ms_of[i]]
    n_timed = sum(len(ms_of[i]) for i in sampled)
    flops_per_launch = float(np.mean([flops_of[i] for i in sampled]))
    avg_ms = float(np.mean([np.mean(ms_of[i]) for i in sampled]))
    achieved = flops_per_launch / (avg_ms * 1e-3) / 1e12
    total_gemm_flops = sum(f for _, _, f, _ in gc)
    if workload == "resnet18":
        metric, unit = f"ResNet-18 fwd images/sec (b{batch},28x28x1,fp32)", "images/s"
        config = {"workload": f"resnet18_forward_b{batch}_28x28x1_fp32"}
        traffic_key = f"resnet18_b{batch}_28x28"
    else:
        metric, unit = f"BERT-base fwd seqs/sec (b{batch},s{seq},fp32)", "seqs/s"
        config = {"workload": f"bert_base_forward_b{batch}_s{seq}_fp32", "variant": variant, "layers": layers,
                  "hidden": cfg.embed_dim, "heads": cfg.num_attention_heads, "ffn": cfg.hidden_dim, "vocab": cfg.num_vocabs,
                  "segment_table_rows": 0 if variant == "reference" else 2}
        traffic_key = f"bert_base_b{batch}_s{seq}" if layers == 12 and variant == "config" else None
    config.update({"replay": "hip_graph" if use_graph else "eager", "launches_per_step": len(prog.calls), "gemm_tflops_whole_step": total_gemm_flops / (ms_per_step * 1e-3) / 1e12})
    traffic = measured_traffic(dom, traffic_key) if traffic_key else None
    res = {
        "metric": metric,
        "value": batch / (ms_per_step * 1e-3),
        "unit": unit,
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": config,
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_FP32_MFMA_TFLOPS,
                     "traffic": traffic, "traffic_source": TRAFFIC_SOURCE if traffic is not None else None,
                     "kernel": dom,
                     "launches_per_step": len(by_name[dom]), "launch_indices_sampled": len(sampled), "launches_timed": n_timed, "avg_launch_ms": avg_ms, "flops_per_launch": flops_per_launch,
                     "shapes_mnkb": sorted({s for _, _, s in by_name[dom]})},
    }
    if use_graph:
        prog.release_graph()
    del prog, logits, model
    if "bert" in keep:
        for k in ("model", "logits", "hidden"):
            keep["bert"].pop(k, None)
    import gc as _gc
    _gc.collect()
    ctx.trim()
    return res, keep


def other_configs(ctx, headline):
    """The other four benchmark configurations, timed in the same run behind the headline: softmax cross-entropy
    [8192,1024] (one fused launch), the 4096^3 GEMM with its bias epilogue, ResNet-18 forward at b128 and the full
    BERT-base forward at b64 x s512.  One entry each: workload, ms_per_step, value/unit and the roofline of its
    dominant kernel."""
    out = []
    ce = next(e for e in headline["roofline_hbm"] if e["workload"] == "softmax_ce") if "roofline_hbm" in headline else None
    if ce is not None:
        out.append({"workload": "softmax_cross_entropy_8192x1024_fp32", "ms_per_step": ce["avg_launch_ms"], "value": 8192 / (ce["avg_launch_ms"] * 1e-3), "unit": "rows/s",
                    "roofline": {"bound": "hbm", "kernel": ce["kernel"], "frac": ce["frac"], "copy_frac": ce["copy_frac"], "avg_launch_ms": ce["avg_launch_ms"],
                                 "bytes_per_launch": ce["bytes"], "achieved": ce["achieved"], "unit": "GB/s"}})
    roof, cfg, _ = time_kernel_workload(ctx, "gemm_bias", 200, 30)
    out.append({"workload": "gemm_bias_4096x4096x4096_fp32", "ms_per_step": roof["avg_launch_ms"], "value": roof["achieved"], "unit": "TFLOP/s",
                "roofline": {"bound": "mfma", "kernel": roof["kernel"], "frac": roof["frac"], "avg_launch_ms": roof["avg_launch_ms"],
                             "flops_per_launch": cfg["flops_per_step"], "achieved": roof["achieved"], "unit": "TFLOP/s", "launches_timed": 200}})
    ctx.trim()
    for workload, batch, seq, steps, warmup in (("resnet18", 128, 0, 50, 10), ("bert", 64, 512, 6, 2)):
        try:
            r, _ = time_model(ctx, workload, "config", batch, seq, 12, steps, warmup, True)
        except Exception as e:  # noqa: BLE001  (the other entries stay)
            out.append({"workload": f"{workload}_b{batch}", "error": f"{type(e).__name__}: {e}"[:400]})
            continue
        rf = r["roofline"]
        out.append({"workload": r["config"]["workload"], "ms_per_step": r["ms_per_step"], "value": r["value"], "unit": r["unit"], "steps": steps,
                    "launches_per_step": r["config"]["launches_per_step"], "gemm_tflops_whole_step": r["config"]["gemm_tflops_whole_step"],
                    "roofline": {"bound": "mfma", "kernel": rf["kernel"], "frac": rf["frac"], "avg_launch_ms": rf["avg_launch_ms"],
                                 "flops_per_launch": rf["flops_per_launch"], "achieved": rf["achieved"], "unit": "TFLOP/s",
                                 "launches_timed": rf["launches_timed"], "shapes_mnkb": rf["shapes_mnkb"]}})
    return out


if __name__ == "__main__":
    main()
