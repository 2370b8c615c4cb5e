"""The chunked allocator behind sg_ctx_create_pooled (use_cache = 1): size classes, splitting and merging, the
capacity on the bytes held, collection and release, against the host-side model of the stated policy
(tests/pool_model.py) and against the invariants any allocator owes (no two live blocks overlap, contents survive
whatever happens around them, the figures of sg_mem_stats add up).  The reference never runs this branch
(context.rs:49), so there is no run of it to compare with: parity with the reference is unpinned here by nature."""
import ctypes as C

import numpy as np
import pytest

import sage_amd as S
from sage_amd import abi
from tests import pool_model as PM
from tests.util import exact

pytestmark = pytest.mark.gpu
MIB = 1 << 20


def say(*a):
    print("[case]", *a, flush=True)


class Dev:
    """sg_alloc / sg_free of one context, with the chunk a pointer belongs to worked out from the addresses seen."""

    def __init__(self, capacity, use_cache=True, use_sub_buffer=True):
        self.ctx = S.Context(capacity=capacity, use_cache=use_cache, use_sub_buffer=use_sub_buffer)
        self.lib = abi.lib()

    def alloc(self, n):
        p = C.c_void_p()
        self.ctx.check(self.lib.sg_alloc(self.ctx.handle, n, C.byref(p)))
        return p.value

    def free(self, p):
        self.ctx.check(self.lib.sg_free(self.ctx.handle, C.c_void_p(p)))

    def stats(self):
        return self.ctx.mem_stats()

    def close(self):
        self.ctx.close()


def test_size_classes_and_chunks():
    d = Dev(capacity=0)
    try:
        say("small requests share a 2 MiB chunk")
        a = d.alloc(4096)
        b = d.alloc(1000)   # rounded to 1024
        c = d.alloc(1)      # rounded to 256
        assert d.stats()["reserved"] == 2 * MIB and d.stats()["used"] == 4096 + 1024 + 256
        assert b == a + 4096 and c == b + 1024, "the request sits in front, the rest of the chunk follows"
        say("a request of 1 MiB and more takes a 20 MiB chunk, one of 10 MiB and more its own size rounded to 2 MiB")
        e = d.alloc(5 * MIB)
        assert d.stats()["reserved"] == 22 * MIB
        f = d.alloc(8 * MIB)
        assert f == e + 5 * MIB and d.stats()["reserved"] == 22 * MIB, "both fit the same 20 MiB chunk"
        g = d.alloc(11 * MIB + 5)
        assert d.stats()["reserved"] == 22 * MIB + 12 * MIB
        # the 12 MiB chunk is handed out whole: the 1 MiB - 256 B behind the request is not worth a block of its own
        assert d.stats()["used"] == 4096 + 1024 + 256 + 13 * MIB + 12 * MIB
        say("freed neighbours merge")
        d.free(a)
        d.free(b)
        a2 = d.alloc(4096 + 1024)
        assert a2 == a, "the merged block serves a request neither part could"
        for p in (a2, c, e, f, g):
            d.free(p)
        s = d.stats()
        assert s["used"] == 0 and s["reserved"] == 34 * MIB and s["peak"] == 34 * MIB
        d.ctx.trim()
        assert d.stats()["reserved"] == 0, "every chunk is whole again and goes back to the device"
    finally:
        d.close()


def test_capacity_bounds_the_chunks_held():
    d = Dev(capacity=64 * MIB)
    try:
        say("three 20 MiB chunks fit under 64 MiB, a fourth does not")
        ps = [d.alloc(19 * MIB) for _ in range(3)]
        assert d.stats()["reserved"] == 60 * MIB
        with pytest.raises(abi.SageError) as e:
            d.alloc(19 * MIB)
        assert e.value.code == abi.ERR_OOM
        needed, total = C.c_uint64(), C.c_uint64()
        d.lib.sg_last_oom(d.ctx.handle, C.byref(needed), C.byref(total))
        assert (needed.value, total.value) == (16 * MIB, 60 * MIB), "check_space on the bytes held (memory.rs:246-255)"
        say("a freed chunk is released to the device when a new chunk of another size needs its room")
        d.free(ps[0])
        q = d.alloc(24 * MIB)  # no free block fits (20 MiB < 24 MiB); 60 + 24 > 64: the free 20 MiB chunk goes first
        assert d.stats()["reserved"] == 64 * MIB
        for p in ps[1:] + [q]:
            d.free(p)
    finally:
        d.close()


def test_old_whole_chunks_are_collected_at_four_fifths():
    d = Dev(capacity=100 * MIB)
    try:
        say("80 MiB in use, one free 12 MiB chunk: the next request that finds no block collects it")
        old = d.alloc(12 * MIB)
        held = [d.alloc(19 * MIB) for _ in range(4)]
        d.free(old)
        more = d.alloc(5 * MIB)  # no free block (the 12 MiB chunk is in the large class and fits!) -> served from it
        assert d.stats()["reserved"] == 92 * MIB, "a fitting free block is used before anything is collected"
        d.free(more)
        big = d.alloc(4 * MIB)   # again from the 12 MiB chunk (split: 8 MiB rest > 1 MiB)
        assert d.stats()["used"] == 4 * 20 * MIB + 4 * MIB
        d.free(big)
        # used = 80 MiB >= 0.8 x 100 MiB; a request no block fits: collection returns the whole free chunk, then a new chunk is taken
        huge = d.alloc(14 * MIB)
        assert d.stats()["reserved"] == 80 * MIB + 14 * MIB
        for p in held + [huge]:
            d.free(p)
    finally:
        d.close()


@pytest.mark.parametrize("seed,capacity,sub", [(0, 0, True), (1, 256 * MIB, True), (2, 96 * MIB, True), (3, 256 * MIB, False)])
def test_random_traces_follow_the_model_and_keep_their_contents(seed, capacity, sub):
    say("random trace", seed, capacity, sub)
    rng = np.random.default_rng(seed)
    d = Dev(capacity=capacity, use_sub_buffer=sub)
    m = PM.Pool(capacity, sub)
    chunk_base = {}   # model chunk id -> device address of its first byte
    live = []         # (pointer, model key, bytes requested, fill value)
    lib, ctx = d.lib, d.ctx
    try:
        for step in range(400):
            if live and (rng.random() < 0.45 or len(live) > 40):
                ptr, key, n, val = live.pop(int(rng.integers(len(live))))
                # the block still holds what was written into it when it was handed out
                words = min(n // 4, 64)
                if words:
                    head = np.zeros(words, np.uint32)
                    ctx.check(lib.sg_memcpy_d2h(ctx.handle, head.ctypes.data_as(C.c_void_p), C.c_void_p(ptr), words * 4))
                    assert (head == val).all(), f"step {step}: contents of a live block changed"
                d.free(ptr)
                m.free(key)
            else:
                kind = rng.random()
                n = int(rng.integers(1, 64 * 1024)) if kind < 0.4 else int(rng.integers(64 * 1024, 3 * MIB)) if kind < 0.8 else int(rng.integers(3 * MIB, 30 * MIB))
                try:
                    chunk, off, size = m.alloc(n)
                except PM.OutOfMemory as oom:
                    with pytest.raises(abi.SageError) as e:
                        d.alloc(n)
                    assert e.value.code == abi.ERR_OOM, f"step {step}: the model is out of memory ({oom}), the library is not"
                    # (the model may have released chunks on the way: forget their addresses)
                    for c in m.chunks_dropped:
                        chunk_base.pop(c, None)
                    m.chunks_dropped.clear()
                    continue
                ptr = d.alloc(n)
                for c in m.chunks_dropped:
                    chunk_base.pop(c, None)
                m.chunks_dropped.clear()
                if chunk in chunk_base:
                    assert ptr == chunk_base[chunk] + off, f"step {step}: block at another offset than the model's ({ptr - chunk_base[chunk]} vs {off})"
                else:
                    chunk_base[chunk] = ptr - off
                assert ptr % 256 == 0
                val = np.uint32(rng.integers(1, 2**32 - 1))
                words = min(n // 4, 64)
                if words:
                    ctx.check(lib.sg_fill_u32(ctx.handle, C.c_void_p(ptr), int(val), words))
                live.append((ptr, (chunk, off), n, val))
            s = d.stats()
            assert (s["used"], s["reserved"], s["peak"]) == (m.used, m.total, m.peak), f"step {step}: {s} vs model {(m.used, m.total, m.peak)}"
            if capacity:
                assert s["reserved"] <= capacity
        # no two live blocks overlap
        spans = sorted((p, p + (max(n, 1) + 255) // 256 * 256) for p, _, n, _ in live)
        assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))
        for ptr, key, _, _ in live:
            d.free(ptr)
            m.free(key)
        assert d.stats()["used"] == 0
        ctx.trim()
        m.trim()
        assert d.stats()["reserved"] == m.total == 0, "after every block came back all chunks are whole and return to the device"
    finally:
        d.close()


def test_a_model_evaluates_the_same_from_the_pool():
    from sage_amd.bert import BertConfig, BertLayer
    say("BERT layers through a pooled context: same bits, graph replay included")
    cfg = BertConfig(256, 100, 64, 512, 2, 4, 1e-12, 0.0, 2)
    x = np.random.default_rng(7).standard_normal((4, 64, 256)).astype(np.float32)
    mask = np.ones((4, 64), np.float32)
    outs = []
    for pooled in (False, True):
        ctx = S.Context(use_cache=pooled)
        try:
            layers = [BertLayer(cfg) for _ in range(2)]
            for i, l in enumerate(layers):
                l.init(ctx, np.random.default_rng(100 + i))
            h = S.Var.new(S.Tensor.from_numpy(ctx, x))
            mk = S.Var.new(S.Tensor.from_numpy(ctx, mask))
            for l in layers:
                h = l.pass_(h, mk)
            eager = h.eval(ctx).numpy()
            prog = S.Program(ctx, [h])
            prog.run()
            replay = prog.outputs[0].numpy()
            prog.capture()
            prog.run()
            prog.run()
            graph = prog.outputs[0].numpy()
            exact(replay, eager, "program replay")
            exact(graph, eager, "graph replay")
            outs.append(eager)
            if pooled:
                s = ctx.mem_stats()
                assert s["reserved"] % (2 * MIB) == 0 and s["reserved"] >= s["used"] > 0
        finally:
            ctx.close()
    exact(outs[1], outs[0], "pooled vs one device allocation per request")
