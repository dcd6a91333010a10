"""Helpers shared by the parity tests."""
import os
import re
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


# Worst err/bound of every comparison made through assert_close, per (test, label with numbers replaced by #):
# [ratio against the bound in force, ratio against the purely elementwise bound rel * |ref|, elements compared,
# elements outside the elementwise bound].  The second is the headroom a tensor would have without the RMS floor
# (inf where a reference element is 0 and the result is not); the last two say how many elements need the floor.
HEADROOM = {}


def record_headroom(what, with_floor, pure, n=0, n_over=0):
    test = os.environ.get("PYTEST_CURRENT_TEST", "").split(" ")[0].split("::")[-1]
    key = (test, re.sub(r"\d+", "#", what))
    old = HEADROOM.get(key, (0.0, 0.0, 0, 0))
    HEADROOM[key] = (max(old[0], with_floor), max(old[1], pure), old[2] + n, old[3] + n_over)


def assert_close(got, ref, rel, what="", sum_abs=None, rms_floor=True):
    """|got - ref| <= rel * max(|ref|, RMS(ref)) elementwise; rms_floor=False: rel * |ref|, the plain relative
    bound.  sum_abs: for results that are sums of many signed terms, the sum of the terms' magnitudes;
    one fp32 ulp of it (2^-24 * sum_abs) is added to the bound -- the floor any fp32 summation
    order has once a long segment cancels to far below its terms.  Returns the worst err/bound."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    assert np.all(np.isfinite(got)) or not np.all(np.isfinite(ref)), f"{what}: non-finite output"
    scale = float(np.sqrt(np.mean(ref ** 2))) if ref.size and rms_floor else 0.0
    extra = 0.0 if sum_abs is None else 2.0 ** -24 * np.asarray(sum_abs, dtype=np.float64)
    bound = rel * np.maximum(np.abs(ref), scale) + 1e-300 + extra
    err = np.abs(got - ref)
    ratio = err / bound
    worst = float(ratio.max()) if ratio.size else 0.0
    pure_ratio = err / (rel * np.abs(ref) + 1e-300 + extra)
    pure = float(pure_ratio.max()) if ratio.size else 0.0
    record_headroom(what, worst, pure, int(ratio.size), int((pure_ratio > 1.0).sum()))
    if worst > 1.0:
        k = np.argmax(ratio)
        raise AssertionError(
            f"{what}: {(ratio > 1).sum()} of {ref.size} elements off; worst got={got.reshape(-1)[k]!r} "
            f"ref={ref.reshape(-1)[k]!r} err/bound={worst:.3g} scale={scale:.3g}")
    return worst


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


def oracle_union_logits(model, table, ids, qs, gamma, cen, regularizer=False, norm=False):
    """Float64 logits [B,U,K] of ids [B,K] against union-branch queries qs = [q1 (, q2)], each [B,U,1,D], as the
    custom_cal_logit bodies compute them before their max over dim 1 (box.py:157-164 and siblings), plus the
    gathered (regularized) rows [B,K,row] they were computed from."""
    b, k = ids.shape
    src = orc.regularizer(table) if regularizer else table
    rows = orc.gather(src, ids).reshape(b, k, -1)
    logit = np.stack([orc.score_forward(model, rows, qs[0][:, j], qs[1][:, j] if len(qs) > 1 else None, gamma, cen,
                                        norm=norm)
                      for j in range(qs[0].shape[1])], axis=1)
    return logit, rows


def oracle_union_grads(model, table, ids, qs, rows, logit, gout, cen, regularizer=False, norm=False):
    """Backward of sum(gout * max over branches of logit): gradient rows [B*K,row] w.r.t. the table rows of the
    pairs and [d/dq1 (, d/dq2)] shaped like qs.  The first maximal branch takes the gradient, as torch.max does;
    with the regularizer clamp(x + 1, 0.05, 1e9) the row gradient is masked where the clamp is active."""
    b, k = ids.shape
    win = np.argmax(logit, axis=1)
    g_rows = np.zeros((b, k, rows.shape[-1]))
    g_qs = [np.zeros_like(q) for q in qs]
    for j in range(logit.shape[1]):
        gj = np.where(win == j, gout, 0.0)
        gr, g1, g2 = orc.score_backward(model, gj, rows, qs[0][:, j], qs[1][:, j] if len(qs) > 1 else None, cen, norm=norm)
        g_rows += gr
        g_qs[0][:, j] = g1
        if len(qs) > 1:
            g_qs[1][:, j] = g2
    g_rows = g_rows.reshape(b * k, -1)
    if regularizer:
        raw = orc.gather(table, ids)
        g_rows = g_rows * ((raw + 1 >= 0.05) & (raw + 1 <= 1e9))
    return g_rows, g_qs


def oracle_adam_step(table, idx_list, grad_list, lr, step, m=None, v=None):
    """unique-merge of all index streams, segment sum, lazy Adam (embed_optimizer.py:39-48,155-163,208-252) in
    float64.  Returns (w, m, v, uniq, merged)."""
    w = table.copy()
    m = np.zeros_like(w) if m is None else m.copy()
    v = np.zeros_like(w) if v is None else v.copy()
    uniq, inverse, _, _ = orc.merge_indices(np.concatenate([np.asarray(i).reshape(-1) for i in idx_list]))
    merged = orc.merge_grads(np.concatenate(grad_list), inverse, uniq.size)
    orc.adam_rows(w, m, v, uniq, merged, lr, step)
    return w, m, v, uniq, merged
