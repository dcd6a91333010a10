"""Helpers shared by the parity tests."""
import zlib

import numpy as np

from oracle import oracle as orc

# Floating-point bar of the scoring path: 1e-5 relative, fp32.  An element is compared
# against max(|reference element|, RMS of the reference tensor): sums over many signed
# terms can cancel to values far below the tensor's scale, where a pure elementwise
# relative bound would ask for more digits than fp32 addition has.
REL_F32 = 1e-5
REL_F64 = 1e-10


def seed(*parts):
    return zlib.crc32(repr(parts).encode())


def assert_close(got, ref, rel, what="", sum_abs=None):
    """sum_abs: for results that are sums of many signed terms, the sum of the terms' magnitudes;
    one fp32 ulp of it (2^-24 * sum_abs) is added to the bound -- the floor any fp32 summation
    order has once a long segment cancels to far below its terms."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    assert np.all(np.isfinite(got)) or not np.all(np.isfinite(ref)), f"{what}: non-finite output"
    scale = float(np.sqrt(np.mean(ref ** 2))) if ref.size else 0.0
    bound = rel * np.maximum(np.abs(ref), scale) + 1e-300
    if sum_abs is not None:
        bound = bound + 2.0 ** -24 * np.asarray(sum_abs, dtype=np.float64)
    err = np.abs(got - ref)
    bad = err > bound
    if bad.any():
        k = np.argmax(err / bound)
        raise AssertionError(
            f"{what}: {bad.sum()} of {ref.size} elements off; worst got={got.reshape(-1)[k]!r} "
            f"ref={ref.reshape(-1)[k]!r} err/bound={(err / bound).reshape(-1)[k]:.3g} scale={scale:.3g}")


def assert_adam_weights(got, want, merged, uniq, lr, what="", floor=0.04):
    """Weights after a lazy Adam step against the oracle's.  Rows `uniq` moved by lr * m_hat / (sqrt(v_hat) + eps):
    that ratio is insensitive to the gradient's size and sensitive to its relative error, which fp32 summation
    bounds only relative to the terms' magnitudes.  So elements whose merged gradient cancelled to below 1e-3 of
    the gradient's RMS may differ by up to the full step (2 lr with a sign flip); every other element must be
    within 1e-5 of max(|weight|, floor).  Returns the worst err/bound over the strictly checked elements."""
    got = np.asarray(got, dtype=np.float64)[uniq]
    want = np.asarray(want, dtype=np.float64)[uniq]
    merged = np.asarray(merged, dtype=np.float64)
    rms = float(np.sqrt(np.mean(merged ** 2))) if merged.size else 0.0
    fragile = np.abs(merged) < 1e-3 * rms
    err = np.abs(got - want)
    bound = REL_F32 * np.maximum(np.abs(want), floor)
    assert err[fragile].size == 0 or err[fragile].max() <= 2.0 * lr, f"{what}: fragile element off by {err[fragile].max()}"
    strict = err[~fragile] / bound[~fragile]
    assert strict.size == 0 or strict.max() <= 1.0, (
        f"{what}: {(strict > 1).sum()} of {strict.size} weights off, worst err/bound={strict.max():.3g}")
    return float(strict.max()) if strict.size else 0.0


def make_inputs(kind, be, ne, bc, nc, dim, rng, scale=1.0):
    """Random operands of one dense operator call (float64 numpy)."""
    mul = 2 if kind in orc.TWO_HALVES else 1
    if kind.startswith("beta"):
        def f(*s):
            x = rng.standard_normal(s)
            return np.clip(1 + np.where(x > 0, x, np.expm1(x)), 0.05, 1e9)
    else:
        def f(*s):
            return rng.standard_normal(s) * scale
    e = f(be, ne, dim * mul)
    q1 = f(bc, nc, dim)
    q2 = None if kind in orc.ONE_QUERY else f(bc, nc, dim)
    return e, q1, q2
