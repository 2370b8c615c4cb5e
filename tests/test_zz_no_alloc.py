"""sg_gemm_noalloc: the GEMM entry point whose split-K workspace is a static per-GPU array.

It must give the bits sg_gemm gives (same kernels, same split), allocate nothing, keep working when
a smaller product follows a larger one in the same array, and refuse a product whose partial
products do not fit.  Runs last in the suite and also passes alone in a fresh process.
"""
import ctypes as C
import gc

import numpy as np
import pytest

import sage_amd as S
from sage_amd import abi
from tests.util import REL_GEMM, close, exact

pytestmark = pytest.mark.gpu


def say(*a):
    print("[case]", *a, flush=True)


def device_free_bytes():
    """Free device memory as the HIP runtime reports it (hipMemGetInfo), asked of the runtime directly: an
    allocation made behind the context's own accounting (a stray hipMalloc in the call) would show here."""
    # The runtime instance libsage_hip.so itself is bound to.  torch bundles a HIP runtime under the same library name:
    # when torch was imported first, the loader binds this library to that copy and no other is mapped; when this
    # library was loaded first, ROCm's own copy is mapped (and torch's, if imported later, is a second instance that
    # knows nothing of this library's allocations).
    abi.lib()
    with open("/proc/self/maps") as f:
        paths = sorted({line.split()[-1] for line in f if "libamdhip64" in line})
    assert paths, "libamdhip64 is not mapped"
    own = [q for q in paths if "/torch/" not in q] or paths
    hip = C.CDLL(own[0])
    free, total = C.c_size_t(), C.c_size_t()
    rc = hip.hipMemGetInfo(C.byref(free), C.byref(total))
    assert rc == 0, f"hipMemGetInfo returned {rc}"
    return free.value


def product(ctx, fn, a, b, bias, res, ta=False, tb=False):
    """relu(op(a).op(b) + bias) + res through one of the two rank-2 GEMM entry points."""
    lib = abi.lib()
    m = a.shape[1] if ta else a.shape[0]
    n = b.shape[0] if tb else b.shape[1]
    ta_, tb_, tbias, tres = (S.Tensor.from_numpy(ctx, x) for x in (a, b, bias, res))
    out = S.Tensor.uninit(ctx, [m, n])
    ac, bc, oc, biasc, resc = ta_.c(), tb_.c(), out.c(), tbias.c(), tres.c()
    epi = abi.sg_gemm_epilogue(1.0, abi.ACT_RELU, abi.ACT_NONE, C.pointer(biasc), C.pointer(resc))
    # (objects of earlier tests that die between the two readings would hand memory back to the device: collect them now)
    gc.collect()
    ctx.sync()
    before = dict(ctx.mem_stats(), device_free=device_free_bytes())
    ctx.check(getattr(lib, fn)(ctx.handle, int(ta), int(tb), C.byref(ac), C.byref(bc), C.byref(oc), C.byref(epi)))
    after = dict(ctx.mem_stats(), device_free=device_free_bytes())
    return out.numpy(), before, after


def test_noalloc_gemm_matches_gemm_twice_second_smaller():
    ctx = S.Context()
    try:
        # both shapes have few output tiles and a long K, so they run split-K through the scratch;
        # the second is smaller in every dimension and reuses the array the first one filled
        for (m, k, n), ta, tb in [((512, 2304, 256), False, False), ((128, 1152, 96), True, False)]:
            say("sg_gemm_noalloc vs sg_gemm", (m, k, n), ta, tb)
            rng = np.random.default_rng(m + k + n)
            a = rng.uniform(-1, 1, (k, m) if ta else (m, k)).astype(np.float32)
            b = rng.uniform(-1, 1, (n, k) if tb else (k, n)).astype(np.float32)
            bias = rng.uniform(-1, 1, (n,)).astype(np.float32)
            res = rng.uniform(-1, 1, (m, n)).astype(np.float32)
            ctx.trim()  # so that sg_gemm's workspace has to come from the device: the control for the probe below
            want, before0, after0 = product(ctx, "sg_gemm", a, b, bias, res, ta, tb)
            got, before, after = product(ctx, "sg_gemm_noalloc", a, b, bias, res, ta, tb)
            exact(got, want, f"sg_gemm_noalloc {m}x{k}x{n}")
            # nothing taken from (or returned to) the context's allocator, nothing new held from the device
            assert after["used"] == before["used"] and after["reserved"] == before["reserved"]
            # ... and nothing taken from the device behind the allocator's back.  The runtime's own bookkeeping (its
            # kernel-argument pool) may grow by a few KiB at any launch, so the bound is a size no workspace here fits in;
            # sg_gemm, whose workspace for the first shape is megabytes, shows that the probe sees an allocation.
            assert before["device_free"] - after["device_free"] < 128 << 10, "the call took memory from the device"
            if (m, k, n) == (512, 2304, 256):
                assert after0["reserved"] > before0["reserved"] and before0["device_free"] - after0["device_free"] >= 1 << 20
            ref = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
            close(got, np.maximum(ref + bias, 0) + res, REL_GEMM, "vs float64")
    finally:
        ctx.close()


def test_noalloc_gemm_without_split_and_over_the_limit():
    ctx = S.Context()
    try:
        say("sg_gemm_noalloc single-pass shape")
        rng = np.random.default_rng(11)
        a = rng.uniform(-1, 1, (1024, 96)).astype(np.float32)
        b = rng.uniform(-1, 1, (96, 768)).astype(np.float32)
        bias = np.zeros(768, np.float32)
        res = np.zeros((1024, 768), np.float32)
        want, _, _ = product(ctx, "sg_gemm", a, b, bias, res)
        got, _, _ = product(ctx, "sg_gemm_noalloc", a, b, bias, res)
        exact(got, want, "single pass")
        # 4 tiles of 128x128 and K = 8192 split 32 ways: 32 * 256 * 256 * 4 B = 8 MiB fits; a product of
        # 1024 x 1024 outputs forced into 32 ranges (128 MiB of partial products) does not
        say("sg_gemm_noalloc over the scratch limit")
        # (the library reads SAGE_GEMM_SPLITK once, when a context is created)
        import os
        os.environ["SAGE_GEMM_SPLITK"] = "32"
        try:
            forced = S.Context()
        finally:
            del os.environ["SAGE_GEMM_SPLITK"]
        try:
            a = rng.uniform(-1, 1, (1024, 4096)).astype(np.float32)
            b = rng.uniform(-1, 1, (4096, 1024)).astype(np.float32)
            with pytest.raises(abi.SageError, match="static scratch"):
                product(forced, "sg_gemm_noalloc", a, b, np.zeros(1024, np.float32), np.zeros((1024, 1024), np.float32))
            # the context still works after the refusal
            got2, _, _ = product(forced, "sg_gemm_noalloc", a[:256, :512].copy(), b[:512, :128].copy(), np.zeros(128, np.float32),
                                 np.zeros((256, 128), np.float32))
        finally:
            forced.close()
        close(got2, np.maximum(a[:256, :512].astype(np.float64) @ b[:512, :128].astype(np.float64), 0), REL_GEMM, "after refusal")
    finally:
        ctx.close()
