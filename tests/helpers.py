"""Shared helpers for the parity tests."""
import numpy as np


def f32_bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def assert_bit_exact(got, want, what=""):
    g, w = f32_bits(got).ravel(), f32_bits(want).ravel()
    assert g.shape == w.shape, f"{what}: shape {g.shape} vs {w.shape}"
    bad = np.nonzero(g != w)[0]
    if bad.size:
        i = int(bad[0])
        raise AssertionError(
            f"{what}: {bad.size} of {g.size} f32 bit patterns differ; first at {i}: "
            f"got {np.asarray(got).ravel()[i]!r} (0x{g[i]:08x}) want {np.asarray(want).ravel()[i]!r} (0x{w[i]:08x})")


# GEMV / GEMM tolerance: "max relative error 1e-3 with fp32 accumulation".
# The error of element j is taken relative to max(|ref_j|, rms(ref)): plain
# relative error wherever the reference is at least of typical size, and
# relative to the typical size for the (arbitrarily small) outputs near zero,
# where a pure ratio is meaningless for any summation order.
REL_TOL = 1e-3


def rel_err(got, ref):
    got = np.asarray(got, dtype=np.float64).ravel()
    ref = np.asarray(ref, dtype=np.float64).ravel()
    rms = float(np.sqrt(np.mean(ref * ref))) if ref.size else 0.0
    den = np.maximum(np.abs(ref), rms if rms > 0 else 1.0)
    return float(np.max(np.abs(got - ref) / den)) if ref.size else 0.0


def assert_close(got, ref, what="", tol=REL_TOL):
    e = rel_err(got, ref)
    assert e <= tol, f"{what}: max relative error {e:.3e} > {tol:.1e}"
    return e
