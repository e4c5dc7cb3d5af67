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


# GEMV / GEMM tolerance: "max relative error 1e-3 with fp32 accumulation".  Three figures are computed:
#   rel_err        max_j |y_j - ref_j| / max(|ref_j|, rms(ref)): plain relative error wherever the reference is
#                  at least of typical size, relative to the typical size for outputs near zero;
#   rel_err_plain  max_j |y_j - ref_j| / |ref_j| over the outputs with |ref_j| > rms(ref) / 10: the plain relative
#                  error of every output that is not small against the typical size (the error of an output does
#                  not shrink with the output -- it is a sum of k rounding errors whose size follows rms(ref) -- so
#                  an output ten times below typical size carries ten times the ratio);
#   rel_err_floor  max_j |y_j - ref_j| / max(|ref_j|, 1e-3 * rms(ref)): the same ratio with a floor a thousand
#                  times lower.  Reported, not gated: among 10^4 outputs the smallest |ref_j| are about
#                  1e-4 * rms, and there two fp32 summation orders of the SAME products already differ by several
#                  1e-3 under this figure (the reference's own sequential fp32 sum is about sqrt(k) * 2^-24 * rms
#                  away from the exact sum; tests/test_oracle_kat.py::test_tolerance_floor_of_fp32_summation
#                  measures it), so it cannot tell a correct kernel from a wrong one.
# A result passes when rel_err <= 1e-3 and rel_err_plain <= 1e-3.  (One kernel is exempt from the second figure at
# short k and says so where it is tested: the fp16 GEMM over the 256-byte Q4_K layout, which contracts q * scale as a
# single fp16 operand.)
REL_TOL = 1e-3


def _flat64(a):
    return np.asarray(a, dtype=np.float64).ravel()


def rel_err(got, ref):
    got, ref = _flat64(got), _flat64(ref)
    if not ref.size:
        return 0.0
    rms = float(np.sqrt(np.mean(ref * ref)))
    den = np.maximum(np.abs(ref), rms if rms > 0 else 1.0)
    return float(np.max(np.abs(got - ref) / den))


def rel_err_plain(got, ref):
    got, ref = _flat64(got), _flat64(ref)
    if not ref.size:
        return 0.0
    rms = float(np.sqrt(np.mean(ref * ref)))
    sel = np.abs(ref) > rms / 10 if rms > 0 else np.zeros(ref.shape, bool)
    return float(np.max(np.abs(got[sel] - ref[sel]) / np.abs(ref[sel]))) if sel.any() else 0.0


def rel_err_floor(got, ref):
    got, ref = _flat64(got), _flat64(ref)
    if not ref.size:
        return 0.0
    rms = float(np.sqrt(np.mean(ref * ref)))
    den = np.maximum(np.abs(ref), 1e-3 * rms if rms > 0 else 1.0)
    return float(np.max(np.abs(got - ref) / den))


def error_report(got, ref):
    return (f"max rel err {rel_err(got, ref):.2e} (floor rms), {rel_err_plain(got, ref):.2e} (plain, |ref| > rms/10), "
            f"{rel_err_floor(got, ref):.2e} (floor 1e-3 rms, reported only)")


def assert_close(got, ref, what="", tol=REL_TOL, plain_tol="same"):
    e = rel_err(got, ref)
    assert e <= tol, f"{what}: max relative error {e:.3e} > {tol:.1e}"
    if plain_tol == "same":
        plain_tol = tol
    if plain_tol is not None:
        p = rel_err_plain(got, ref)
        assert p <= plain_tol, f"{what}: max plain relative error {p:.3e} > {plain_tol:.1e} (outputs with |ref| > rms / 10)"
    return e
