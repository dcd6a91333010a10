"""TEST INFRASTRUCTURE ONLY: numpy front end of the CPU oracle (oracle/liboracle.so).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module.  Nothing under smore_amd/ does.

Reference lines restated by each function are cited in oracle_body.inc /
smore_oracle.c.  The reference holds no golden vectors for this path (its tests
only print numbers), and its own implementation is CUDA-only, so each oracle
function is pinned by an independent check in tests/test_oracle_pinning.py:

  function                  pinned by
  ------------------------  ----------------------------------------------------
  digamma / trigamma        scipy.special.digamma / polygamma(1), psi(1) = -gamma,
                            psi'(1) = pi^2/6, the recurrences psi(x+1)-psi(x)=1/x
  lgamma                    scipy.special.gammaln, lgamma(n) = log((n-1)!)
  dist_forward (all kinds)  closed forms written with numpy abs/maximum/minimum/
                            sqrt, torch.distributions.kl._kl_beta_beta, brute
                            force of the broadcast index rule on tiny shapes
  dist_backward             torch.autograd of those closed forms at tie-free fp64
                            inputs, central finite differences, hand-built tie
                            cases for the kernel's subgradient conventions
  gather                    numpy fancy indexing
  regularizer               numpy clip
  merge_indices             numpy.unique(return_inverse=True), stable argsort
  merge_grads               numpy.add.at
  adam_rows                 torch.optim.Adam when every row is touched each
                            step; untouched rows bit-identical; hand-computed
                            first step; squeeze variant by closed form
  sgd / adagrad / rmsprop   torch.optim.SGD / Adagrad / RMSprop(alpha=0.99) when
                            every row is touched; squeeze variants by closed form
  unit_halves (+backward)   torch.nn.functional.normalize (the routine the reference calls) and
                            its autograd on each half, unit length of the result, orthogonality
                            of the gradient to the row, central finite differences, the
                            below-eps branch by hand
  score / train_step        composition only (gamma - dist, gamma + similarity, chain rule of sqrt)
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

KINDS = {
    "l1": 0, "l2": 1, "box_out": 2, "box_in": 3, "rotate": 4, "beta_kl": 5,
    "complex": 6, "distmult": 7, "beta_l2": 8, "beta_fisher_approx": 9,
}
TWO_HALVES = {"rotate", "complex", "beta_kl", "beta_l2", "beta_fisher_approx"}
ONE_QUERY = {"l1", "l2", "distmult"}


def build():
    subprocess.run(["make", "-C", _HERE, "-s", "liboracle.so"], check=True)


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
        _LIB.orc_merge_indices.restype = ctypes.c_int64
    return _LIB


def _sfx(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float64:
        return "f64", ctypes.c_double
    if dtype == np.float32:
        return "f32", ctypes.c_float
    raise TypeError(dtype)


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _sz(x):
    return ctypes.c_size_t(int(x))


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def special(name, x, dtype=np.float64):
    """name in {digamma, trigamma, lgamma}, elementwise."""
    sfx, _ = _sfx(dtype)
    x = _c(x, dtype)
    out = np.empty_like(x)
    which = {"digamma": 0, "trigamma": 1, "lgamma": 2}[name]
    getattr(lib(), f"orc_special_{sfx}")(which, _p(x), _sz(x.size), _p(out))
    return out


def _shapes(kind, ent, q1, q2):
    assert ent.ndim == 3 and q1.ndim == 3
    be, ne, de = ent.shape
    bc, nc, dim = q1.shape
    mul = 2 if kind in TWO_HALVES else 1
    assert de == dim * mul, (de, dim, mul)
    if q2 is not None:
        assert q2.shape == q1.shape
    assert be % bc == 0 or bc % be == 0
    assert ne % nc == 0 or nc % ne == 0
    return be, ne, bc, nc, dim, max(be, bc), max(ne, nc)


def dist_forward(kind, ent, q1, q2=None, dtype=np.float64):
    """out[i,j] = sum_d f(ent[i%be, j%ne], q[i%bc, j%nc]); 3-D inputs."""
    sfx, _ = _sfx(dtype)
    ent, q1 = _c(ent, dtype), _c(q1, dtype)
    q2 = None if q2 is None else _c(q2, dtype)
    be, ne, bc, nc, dim, bsize, num = _shapes(kind, ent, q1, q2)
    dst = np.empty((bsize, num), dtype=dtype)
    rc = getattr(lib(), f"orc_dist_forward_{sfx}")(
        KINDS[kind], _p(ent), _p(q1), _p(q2), _p(dst),
        _sz(bsize), _sz(num), _sz(be), _sz(ne), _sz(bc), _sz(nc), _sz(dim))
    assert rc == 0
    return dst


def dist_backward(kind, gout, ent, q1, q2=None, dtype=np.float64):
    """Returns (gent, gq1, gq2-or-None), each the shape of its input."""
    sfx, _ = _sfx(dtype)
    ent, q1, gout = _c(ent, dtype), _c(q1, dtype), _c(gout, dtype)
    q2 = None if q2 is None else _c(q2, dtype)
    be, ne, bc, nc, dim, bsize, num = _shapes(kind, ent, q1, q2)
    assert gout.shape == (bsize, num)
    gent = np.empty_like(ent)
    gq1 = np.empty_like(q1)
    gq2 = None if q2 is None else np.empty_like(q2)
    rc = getattr(lib(), f"orc_dist_backward_{sfx}")(
        KINDS[kind], _p(gout), _p(ent), _p(q1), _p(q2), _p(gent), _p(gq1), _p(gq2),
        _sz(bsize), _sz(num), _sz(be), _sz(ne), _sz(bc), _sz(nc), _sz(dim))
    assert rc == 0
    return gent, gq1, gq2


def gather(table, idx, dtype=None):
    dtype = table.dtype if dtype is None else dtype
    sfx, _ = _sfx(dtype)
    table = _c(table, dtype)
    idx = _c(idx, np.int64).reshape(-1)
    out = np.empty((idx.size, table.shape[1]), dtype=dtype)
    rc = getattr(lib(), f"orc_gather_{sfx}")(
        _p(table), _sz(table.shape[0]), _sz(table.shape[1]), _p(idx), _sz(idx.size), _p(out))
    if rc != 0:
        raise IndexError("entity id out of range")
    return out


def regularizer(x, base_add=1.0, lo=0.05, hi=1e9, dtype=np.float64):
    sfx, ct = _sfx(dtype)
    x = _c(x, dtype)
    out = np.empty_like(x)
    getattr(lib(), f"orc_regularizer_{sfx}")(_p(x), _sz(x.size), ct(base_add), ct(lo), ct(hi), _p(out))
    return out


def unit_halves(rows, dtype=np.float64, eps=1e-12, halves=2):
    """Each half of the last axis scaled to unit L2 length, x / max(|x|, eps): what ComplexReasoning does to an
    entity row before complex_sim when its mode names 'norm' (models/complex.py:142-146; embed_norm = Normalizer,
    common/modules.py:38-40 = F.normalize(p=2, dim=-1), whose eps is 1e-12).  halves = 1: the whole row, DistMult's
    'norm' mode (models/distmult.py:129-130)."""
    rows = np.asarray(rows, dtype=dtype)
    h = rows.shape[-1] // halves
    out = np.empty_like(rows)
    for sl in [slice(i * h, (i + 1) * h) for i in range(halves)]:
        x = rows[..., sl]
        n = np.maximum(np.sqrt((x * x).sum(axis=-1, keepdims=True)), dtype(eps))
        out[..., sl] = x / n
    return out


def unit_halves_backward(rows, gout, dtype=np.float64, eps=1e-12, halves=2):
    """Gradient w.r.t. rows of sum(gout * unit_halves(rows)): per half (g - x_n (x_n . g)) / |x| where |x| > eps,
    g / eps below (the denominator is then the constant eps)."""
    rows = np.asarray(rows, dtype=dtype)
    gout = np.asarray(gout, dtype=dtype)
    h = rows.shape[-1] // halves
    out = np.empty_like(rows)
    for sl in [slice(i * h, (i + 1) * h) for i in range(halves)]:
        x, g = rows[..., sl], gout[..., sl]
        n = np.sqrt((x * x).sum(axis=-1, keepdims=True))
        live = n > eps
        safe = np.where(live, n, dtype(1.0))
        xn = x / safe
        proj = (g - xn * (xn * g).sum(axis=-1, keepdims=True)) / safe
        out[..., sl] = np.where(live, proj, g / dtype(eps))
    return out


def merge_indices(idx):
    """Returns (uniq[U], inverse[P], order[P], seg_start[U+1]).

    uniq is sorted ascending; order lists pair positions grouped by id, ties in
    ascending pair order; seg_start[u]..seg_start[u+1] is segment u in order[].
    """
    idx = _c(idx, np.int64).reshape(-1)
    p = idx.size
    uniq = np.empty(p, dtype=np.int64)
    inverse = np.empty(p, dtype=np.int64)
    order = np.empty(p, dtype=np.int64)
    seg = np.empty(p + 1, dtype=np.int64)
    u = lib().orc_merge_indices(_p(idx), _sz(p), _p(uniq), _p(inverse), _p(order), _p(seg))
    return uniq[:u].copy(), inverse, order, seg[: u + 1].copy()


def merge_grads(grad, inverse, n_uniq, dtype=np.float64):
    sfx, _ = _sfx(dtype)
    grad = _c(grad, dtype)
    inverse = _c(inverse, np.int64)
    merged = np.empty((n_uniq, grad.shape[1]), dtype=dtype)
    getattr(lib(), f"orc_merge_grads_{sfx}")(
        _p(grad), _p(inverse), _sz(grad.shape[0]), _sz(grad.shape[1]), _sz(n_uniq), _p(merged))
    return merged


def adam_rows(w, m, v, uniq, merged, lr, step, beta1=0.9, beta2=0.999, eps=1e-8, squeeze=False):
    """In-place lazy Adam on rows uniq of w, m, v (all C-contiguous, same dtype)."""
    sfx, _ = _sfx(w.dtype)
    assert w.flags.c_contiguous and m.flags.c_contiguous and v.flags.c_contiguous
    assert m.dtype == w.dtype and v.dtype == w.dtype
    uniq = _c(uniq, np.int64)
    merged = _c(merged, w.dtype)
    getattr(lib(), f"orc_adam_rows_{sfx}")(
        _p(w), _p(m), _p(v), _p(uniq), _p(merged), _sz(uniq.size), _sz(w.shape[1]),
        ctypes.c_double(lr), ctypes.c_double(beta1), ctypes.c_double(beta2), ctypes.c_double(eps),
        ctypes.c_long(int(step)), ctypes.c_int(1 if squeeze else 0))


def sgd_rows(w, uniq, merged, lr):
    sfx, _ = _sfx(w.dtype)
    uniq, merged = _c(uniq, np.int64), _c(merged, w.dtype)
    getattr(lib(), f"orc_sgd_rows_{sfx}")(_p(w), _p(uniq), _p(merged), _sz(uniq.size), _sz(w.shape[1]),
                                          ctypes.c_double(lr))


def adagrad_rows(w, state, uniq, merged, lr, eps=1e-8, squeeze=False):
    sfx, _ = _sfx(w.dtype)
    uniq, merged = _c(uniq, np.int64), _c(merged, w.dtype)
    assert state.flags.c_contiguous and state.dtype == w.dtype
    getattr(lib(), f"orc_adagrad_rows_{sfx}")(_p(w), _p(state), _p(uniq), _p(merged), _sz(uniq.size), _sz(w.shape[1]),
                                              ctypes.c_double(lr), ctypes.c_double(eps), ctypes.c_int(int(squeeze)))


def rmsprop_rows(w, state, uniq, merged, lr, alpha=0.99, eps=1e-8, squeeze=False):
    sfx, _ = _sfx(w.dtype)
    uniq, merged = _c(uniq, np.int64), _c(merged, w.dtype)
    assert state.flags.c_contiguous and state.dtype == w.dtype
    getattr(lib(), f"orc_rmsprop_rows_{sfx}")(_p(w), _p(state), _p(uniq), _p(merged), _sz(uniq.size), _sz(w.shape[1]),
                                              ctypes.c_double(lr), ctypes.c_double(alpha), ctypes.c_double(eps),
                                              ctypes.c_int(int(squeeze)))


def sample_loss(pos, neg, mask=None, weight=None, temperature=0.0, scale=0.5, dtype=np.float64):
    """Sample loss of train_process.py:194-213 and its gradient w.r.t. the logits.
    Returns (pos_loss, neg_loss, gpos [B], gneg [B,K]); the gradients are those of (pos_loss + neg_loss) * scale."""
    sfx, _ = _sfx(dtype)
    pos, neg = _c(pos, dtype).reshape(-1), _c(neg, dtype)
    b, k = neg.shape
    assert pos.size == b
    mask = None if mask is None else _c(mask, dtype)
    weight = None if weight is None else _c(weight, dtype).reshape(-1)
    out, gpos, gneg = np.zeros(2, dtype), np.zeros(b, dtype), np.zeros((b, k), dtype)
    getattr(lib(), f"orc_sample_loss_{sfx}")(_p(pos), _p(neg), _p(mask) if mask is not None else None,
                                             _p(weight) if weight is not None else None, _sz(b), _sz(k),
                                             ctypes.c_double(temperature), ctypes.c_double(scale), _p(out), _p(gpos),
                                             _p(gneg))
    return float(out[0]), float(out[1]), gpos, gneg


def filtered_ranks(scores, easy, hard):
    """Filtered ranks (1-based) of one query's answers among all entities, train_process.py:124-145:
    ranking = position in the descending argsort of the logits (equal logits: lower id first), and an
    answer's filtered rank is its position minus the number of answers (easy or hard) placed before it.
    scores [N]; easy, hard: disjoint id sequences.  Returns (ranks of hard, ranks of easy) in the given order."""
    scores = np.asarray(scores)
    order = np.argsort(-scores, kind="stable")
    ranking = np.empty(scores.shape[0], dtype=np.int64)
    ranking[order] = np.arange(scores.shape[0])
    ans = np.array(list(easy) + list(hard), dtype=np.int64)
    pos = ranking[ans] if ans.size else np.zeros(0, np.int64)
    before = (pos[None, :] < pos[:, None]).sum(axis=1) if ans.size else pos
    filt = pos - before + 1
    return filt[len(easy):], filt[: len(easy)]


def candidate_ranks(logit, neg, n_hard):
    """Evaluation against sampled candidates, train_process.py:118-128 and 141-147.  logit [C]: the logits of one
    query's candidates neg [C] (padding -1 scored as entity 0, :120); the bias -1e6 is added where neg == -1 (:119,
    :123); ranking = position in the descending argsort of the biased logits (equal logits: lower position first);
    the first n_hard candidates are the hard answers, and the filtered rank of one is its position minus the
    number of hard answers before it, plus 1.  Returns (biased logits, ranking [C], filtered ranks [n_hard] in the
    order given)."""
    logit = np.asarray(logit)
    biased = logit + np.where(np.asarray(neg) == -1, logit.dtype.type(-1e6), logit.dtype.type(0))
    order = np.argsort(-biased, kind="stable")
    ranking = np.empty(biased.shape[0], dtype=np.int64)
    ranking[order] = np.arange(biased.shape[0])
    pos = ranking[:n_hard]
    before = (pos[None, :] < pos[:, None]).sum(axis=1) if n_hard else pos
    return biased, ranking, pos - before + 1


# ---- composition: the score of each model and one training step -------------------------------

MODELS = ("l1", "l2", "box", "rotate", "beta_kl", "complex", "distmult")
SIMILARITY = ("complex", "distmult")


def score_forward(model, rows, q1, q2=None, gamma=0.0, cen=0.0, dtype=np.float64, norm=False):
    """rows [B,K,De], q [B,1,D] -> logit [B,K] as the custom_cal_logit bodies compute it
    (models/vec.py:85-90, box.py:157-164, rotate.py:137-142, beta.py:303-308) with one
    union branch; l2 takes the square root outside the operator (dist_func/l2_dist.py:59-62).
    norm (complex: the halves of every entity row at unit length first, complex.py:142-146; distmult: the whole
    row, distmult.py:129-130)."""
    if norm:
        assert model in SIMILARITY
        rows = unit_halves(rows, dtype, halves=2 if model == "complex" else 1)
    if model == "box":
        d = dist_forward("box_out", rows, q1, q2, dtype) + cen * dist_forward("box_in", rows, q1, q2, dtype)
    elif model == "l2":
        d = np.sqrt(dist_forward("l2", rows, q1, None, dtype))
    elif model in SIMILARITY:   # models/complex.py:140-148, distmult.py: the logit is the similarity itself
        return (gamma + dist_forward(model, rows, q1, q2, dtype)).astype(dtype)
    else:
        d = dist_forward(model, rows, q1, q2, dtype)
    return (gamma - d).astype(dtype)


def score_backward(model, gscore, rows, q1, q2=None, cen=0.0, dtype=np.float64, norm=False):
    """Gradients of sum(gscore * score) w.r.t. rows, q1, q2."""
    gscore = np.asarray(gscore, dtype=dtype)
    if norm:
        assert model in SIMILARITY
        halves = 2 if model == "complex" else 1
        gn, gq1, gq2 = dist_backward(model, gscore, unit_halves(rows, dtype, halves=halves), q1, q2, dtype)
        return unit_halves_backward(rows, gn, dtype, halves=halves), gq1, gq2
    if model == "box":
        a = dist_backward("box_out", -gscore, rows, q1, q2, dtype)
        b = dist_backward("box_in", -cen * gscore, rows, q1, q2, dtype)
        return tuple(x + y for x, y in zip(a, b))
    if model == "l2":
        d2 = dist_forward("l2", rows, q1, None, dtype)
        g = -gscore / (2.0 * np.sqrt(d2))
        return dist_backward("l2", g.astype(dtype), rows, q1, None, dtype)
    if model in SIMILARITY:
        return dist_backward(model, gscore, rows, q1, q2, dtype)
    return dist_backward(model, -gscore, rows, q1, q2, dtype)


def train_step(model, table, m, v, idx, q1, q2, gscore, gamma, cen, lr, step, dtype=np.float64,
               squeeze=False, apply_adam=True, norm=False):
    """One pass in the order of training/train_process.py:172-220 with the loss replaced by
    a given upstream gradient: gather, score, backward, unique-merge, segment sum, lazy Adam.
    table/m/v are updated in place.  Returns a dict of everything in between."""
    b, k = idx.shape
    rows = gather(table, idx, dtype).reshape(b, k, -1)
    score = score_forward(model, rows, q1, q2, gamma, cen, dtype, norm)
    grows, gq1, gq2 = score_backward(model, gscore, rows, q1, q2, cen, dtype, norm)
    uniq, inverse, order, seg_start = merge_indices(idx)
    merged = merge_grads(grows.reshape(b * k, -1), inverse, uniq.size, dtype)
    if apply_adam:
        adam_rows(table, m, v, uniq, merged, lr, step, squeeze=squeeze)
    return dict(score=score, gq1=gq1, gq2=gq2, uniq=uniq, inverse=inverse, order=order,
                seg_start=seg_start, merged=merged)
