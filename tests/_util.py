"""Shared helpers for the parity tests (seeded inputs, tolerances)."""
import numpy as np

GOLDEN = __import__("os").path.join(__import__("os").path.dirname(__file__), "golden")

# north_star tolerance for matmul outputs: 1e-3 relative to the f64 result
# (fp32 accumulate), element by element.  A dot product can cancel to ~0, where a
# relative bound means nothing, so an absolute floor of 1e-4 of the output RMS is
# added (observed errors are ~3e-6 of the RMS: fp32 accumulation noise).
REL_TOL = 1e-3
ABS_FLOOR = 1e-4


def assert_matmul_close(got, ref64, what=""):
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    ref = np.asarray(ref64, dtype=np.float64).reshape(-1)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    rms = float(np.sqrt(np.mean(ref * ref))) if ref.size else 0.0
    err = np.abs(got - ref)
    bound = REL_TOL * np.abs(ref) + ABS_FLOOR * rms
    bad = err > bound
    if bad.any():
        i = int(np.argmax(err - bound))
        raise AssertionError(f"{what}: {int(bad.sum())}/{ref.size} outside 1e-3 rel; worst idx {i}: "
                             f"got {got[i]!r} ref {ref[i]!r} (rms {rms:.4g})")
    if rms > 0:
        cos = float(got @ ref / (np.linalg.norm(got) * np.linalg.norm(ref)))
        assert cos >= 0.9999, f"{what}: cosine {cos}"
    return float(err.max() / rms) if rms > 0 else 0.0


# The Q4_K tile GEMM (m > 8) rounds every dequantised weight once to f16 (2^-12 relative), as the
# reference's mul_mm kernels do with their half-precision weight tile; bf16 activations stay exact,
# f32 activations are rounded to f16 as well.  Its gate is the one the scope table states for matmul
# outputs, max|err| / max|ref| <= 1e-3 with cosine >= 0.9999, plus an element-wise bound of
# 1e-3 |ref| + 3e-3 rms (observed: rms error 2-3e-4 of the output rms, worst element 1.5e-3 rms).
F16_TILE_ABS = 3e-3


def assert_matmul_close_f16_tile(got, ref64, what=""):
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    ref = np.asarray(ref64, dtype=np.float64).reshape(-1)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    if not ref.size:
        return 0.0
    rms = float(np.sqrt(np.mean(ref * ref)))
    err = np.abs(got - ref)
    peak = float(np.abs(ref).max())
    if peak == 0.0:
        assert not got.any(), f"{what}: reference is zero, output is not"
        return 0.0
    assert err.max() <= REL_TOL * peak, f"{what}: max|err| {err.max():.4g} > 1e-3 max|ref| {peak:.4g}"
    bound = REL_TOL * np.abs(ref) + F16_TILE_ABS * rms
    bad = err > bound
    assert not bad.any(), f"{what}: {int(bad.sum())}/{ref.size} outside 1e-3 |ref| + 3e-3 rms (rms {rms:.4g})"
    assert float(np.sqrt(np.mean(err * err))) <= 5e-4 * rms, f"{what}: rms error above 5e-4 of the output rms"
    cos = float(got @ ref / (np.linalg.norm(got) * np.linalg.norm(ref)))
    assert cos >= 0.9999, f"{what}: cosine {cos}"
    return float(err.max() / rms)


def weights(seed, n, k, sigma=0.02):
    """Seeded N(0, sigma) f32 weight [n, k] (the benchmark's weight distribution)."""
    return (np.random.default_rng(seed).standard_normal((n, k), dtype=np.float32) * np.float32(sigma))


def acts(seed, m, k):
    return np.random.default_rng(seed).standard_normal((m, k), dtype=np.float32)
