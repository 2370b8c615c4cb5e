"""Shared helpers of the parity tests."""
import numpy as np

REL_MAP = 1e-4     # elementwise and reductions (fp32)
REL_GEMM = 1e-3    # GEMM and end-to-end model output


def close(a, b, rel, what=""):
    """|a-b| <= rel * max(|b|, scale) elementwise, scale = RMS of b (absolute floor for values near 0)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    assert a.shape == b.shape, f"{what}: shape {a.shape} vs {b.shape}"
    fin = np.isfinite(b)
    assert np.array_equal(np.isfinite(a), fin), f"{what}: finiteness differs"
    assert np.array_equal(np.isnan(a), np.isnan(b)), f"{what}: NaN pattern differs"
    inf = np.isinf(b)
    assert np.array_equal(a[inf], b[inf]), f"{what}: infinities differ"
    if not fin.any():
        return
    scale = float(np.sqrt(np.mean(b[fin] ** 2))) or 1.0
    err = np.abs(a[fin] - b[fin])
    tol = rel * np.maximum(np.abs(b[fin]), scale)
    worst = float(np.max(err / tol))
    assert worst <= 1.0, f"{what}: worst error {worst:.3g} x tolerance (rel {rel})"


def exact(a, b, what=""):
    a, b = np.asarray(a), np.asarray(b)
    assert a.shape == b.shape, f"{what}: shape {a.shape} vs {b.shape}"
    assert a.dtype == b.dtype, f"{what}: dtype {a.dtype} vs {b.dtype}"
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), f"{what}: not bit-exact"
