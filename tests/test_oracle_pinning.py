"""Pins the CPU oracle against independent facts (library routines, closed forms,
autograd of the textbook expressions, brute force) before anything is compared
with it.  The reference holds no golden vectors for this path."""
import math
import zlib

import numpy as np
import pytest
import scipy.special as sp
import torch

from oracle import oracle as orc

RNG = np.random.default_rng(7)


def _seed(*parts):
    return zlib.crc32(repr(parts).encode())


# ---------------------------------------------------------------- special functions

def test_digamma_trigamma_lgamma_against_scipy():
    x = np.concatenate([RNG.uniform(0.05, 12.0, 4000), RNG.uniform(12.0, 500.0, 500),
                        [0.05, 0.5, 1.0, 2.0, 9.999, 10.0, 10.001, 1e6]])
    assert np.allclose(orc.special("digamma", x), sp.digamma(x), rtol=1e-12, atol=1e-12)
    # the reference's trigamma series (6 recurrence steps + 4-term tail) is itself only 1e-8 accurate
    assert np.allclose(orc.special("trigamma", x), sp.polygamma(1, x), rtol=2e-8, atol=0)
    assert np.allclose(orc.special("lgamma", x), sp.gammaln(x), rtol=1e-13, atol=1e-13)


def test_special_known_values_and_recurrences():
    assert abs(orc.special("digamma", [1.0])[0] + np.euler_gamma) < 1e-14
    assert abs(orc.special("digamma", [10.0])[0] - 2.2517525890667211) < 1e-15
    assert abs(orc.special("trigamma", [1.0])[0] - math.pi ** 2 / 6) < 1e-8
    x = RNG.uniform(0.05, 30.0, 1000)
    assert np.allclose(orc.special("digamma", x + 1) - orc.special("digamma", x), 1 / x, rtol=0, atol=1e-12)
    assert np.allclose(orc.special("trigamma", x + 1) - orc.special("trigamma", x), -1 / x ** 2, rtol=1e-7, atol=1e-9)
    n = np.arange(1, 20, dtype=np.float64)
    assert np.allclose(orc.special("lgamma", n), [math.log(math.factorial(int(k) - 1)) for k in n], atol=1e-12)
    # negative arguments: reflection branch of the reference series
    xn = np.array([-0.5, -1.5, -2.25, 0.25, 0.4])
    assert np.allclose(orc.special("digamma", xn), sp.digamma(xn), rtol=1e-12)
    assert np.allclose(orc.special("trigamma", xn),
                       torch.polygamma(1, torch.tensor(xn, dtype=torch.float64)).numpy(), rtol=1e-7)
    assert np.isinf(orc.special("digamma", [0.0])[0]) and np.isnan(orc.special("digamma", [-2.0])[0])


def test_f32_special_close_to_f64():
    x = RNG.uniform(0.05, 40.0, 2000)
    for name, tol in (("digamma", 3e-6), ("trigamma", 3e-6), ("lgamma", 3e-6)):
        a = orc.special(name, x.astype(np.float32), np.float32).astype(np.float64)
        b = orc.special(name, x.astype(np.float32).astype(np.float64))
        assert np.all(np.abs(a - b) <= tol * np.maximum(1.0, np.abs(b))), name


# ---------------------------------------------------------------- forward closed forms

def _halves(e):
    d = e.shape[-1] // 2
    return e[..., :d], e[..., d:]


def closed_form(kind, e, q1, q2):
    """Textbook expressions with numpy broadcasting on [be,ne,De] x [bc,nc,D]."""
    if kind == "l1":
        return np.abs(e - q1).sum(-1)
    if kind == "l2":
        return ((e - q1) ** 2).sum(-1)
    if kind == "box_out":
        return np.maximum(np.abs(e - q1) - q2, 0).sum(-1)
    if kind == "box_in":
        return np.abs(np.minimum(np.abs(e - q1), q2)).sum(-1)
    if kind == "rotate":
        a, b = _halves(e)
        return np.sqrt((a - q1) ** 2 + (b - q2) ** 2 + 1e-20).sum(-1)
    if kind == "complex":
        a, b = _halves(e)
        return (a * q1 + b * q2).sum(-1)
    if kind == "distmult":
        return (e * q1).sum(-1)
    if kind == "beta_l2":
        a, b = _halves(e)
        return 0.5 * ((a - q1) ** 2 + (b - q2) ** 2).sum(-1)
    if kind == "beta_kl":
        a, b = _halves(e)
        sp_, sq = a + b, q1 + q2
        t = (sp.gammaln(q1) + sp.gammaln(q2) + sp.gammaln(sp_) - sp.gammaln(a) - sp.gammaln(b) - sp.gammaln(sq)
             + (a - q1) * sp.digamma(a) + (b - q2) * sp.digamma(b) + (sq - sp_) * sp.digamma(sp_))
        return t.sum(-1)
    if kind == "beta_fisher_approx":
        a, b = _halves(e)
        ta, tb, tab = sp.polygamma(1, a), sp.polygamma(1, b), -sp.polygamma(1, a + b)
        da, db = a - q1, b - q2
        return 0.5 * ((ta + tab) * da ** 2 + 2 * tab * da * db + (tb + tab) * db ** 2).sum(-1)
    raise KeyError(kind)


def make_inputs(kind, be, ne, bc, nc, dim, rng, positive=False):
    mul = 2 if kind in orc.TWO_HALVES else 1
    if kind.startswith("beta"):
        f = lambda *s: np.clip(1 + np.where((x := rng.standard_normal(s)) > 0, x, np.expm1(x)), 0.05, 1e9)
    else:
        f = lambda *s: rng.standard_normal(s)
    e = f(be, ne, dim * mul)
    q1 = f(bc, nc, dim)
    q2 = None if kind in orc.ONE_QUERY else f(bc, nc, dim)
    if kind.startswith("box") and positive:
        q2 = np.abs(q2)
    return e, q1, q2


LAYOUTS = [  # (be, ne, bc, nc): every caller situation the operator must accept
    (6, 5, 6, 1),   # per-query negatives
    (1, 7, 4, 1),   # shared negatives
    (5, 1, 5, 1),   # positives
    (1, 9, 1, 1),   # eval against all entities
    (4, 1, 4, 6),   # reverse queries (ne=1 < nc)
    (6, 1, 1, 5),   # the reference's smoke-test layout
    (6, 4, 3, 2),   # both sides broadcast by modulo
]


@pytest.mark.parametrize("kind", list(orc.KINDS))
@pytest.mark.parametrize("layout", LAYOUTS)
def test_forward_matches_closed_form(kind, layout):
    be, ne, bc, nc = layout
    rng = np.random.default_rng(_seed(kind, layout))
    e, q1, q2 = make_inputs(kind, be, ne, bc, nc, 11, rng)
    got = orc.dist_forward(kind, e, q1, q2)
    bsize, num = max(be, bc), max(ne, nc)
    # modulo broadcast rule of the launch loop, spelled out by brute force
    ii, jj = np.meshgrid(np.arange(bsize), np.arange(num), indexing="ij")
    eb = e[ii % be, jj % ne]
    q1b = q1[ii % bc, jj % nc]
    q2b = None if q2 is None else q2[ii % bc, jj % nc]
    want = closed_form(kind, eb, q1b, q2b)
    tol = 3e-8 if "fisher" in kind else 1e-11
    assert np.allclose(got, want, rtol=tol, atol=tol)


def test_beta_kl_is_torch_kl_beta_beta():
    rng = np.random.default_rng(3)
    e, q1, q2 = make_inputs("beta_kl", 8, 6, 8, 1, 16, rng)
    from torch.distributions import Beta
    from torch.distributions.kl import _kl_beta_beta
    a, b = _halves(torch.from_numpy(e))
    kl = _kl_beta_beta(Beta(a, b), Beta(torch.from_numpy(q1), torch.from_numpy(q2))).sum(-1).numpy()
    assert np.allclose(orc.dist_forward("beta_kl", e, q1, q2), kl, rtol=1e-11, atol=1e-11)
    assert np.all(kl > -1e-9)


# ---------------------------------------------------------------- backward

def torch_form(kind, e, q1, q2):
    if kind == "l1":
        return (e - q1).abs().sum(-1)
    if kind == "l2":
        return ((e - q1) ** 2).sum(-1)
    if kind == "box_out":
        return torch.relu((e - q1).abs() - q2).sum(-1)
    if kind == "box_in":
        return torch.minimum((e - q1).abs(), q2).abs().sum(-1)
    a, b = torch.chunk(e, 2, dim=-1) if kind in orc.TWO_HALVES else (e, None)
    if kind == "rotate":
        return torch.sqrt((a - q1) ** 2 + (b - q2) ** 2 + 1e-20).sum(-1)
    if kind == "complex":
        return (a * q1 + b * q2).sum(-1)
    if kind == "distmult":
        return (e * q1).sum(-1)
    if kind == "beta_l2":
        return 0.5 * ((a - q1) ** 2 + (b - q2) ** 2).sum(-1)
    if kind == "beta_kl":
        sp_, sq = a + b, q1 + q2
        return (torch.lgamma(q1) + torch.lgamma(q2) + torch.lgamma(sp_) - torch.lgamma(a) - torch.lgamma(b)
                - torch.lgamma(sq) + (a - q1) * torch.digamma(a) + (b - q2) * torch.digamma(b)
                + (sq - sp_) * torch.digamma(sp_)).sum(-1)
    if kind == "beta_fisher_approx":
        with torch.no_grad():  # the reference treats the trigamma weights as constants
            ta, tb, tab = a.polygamma(1), b.polygamma(1), -(a + b).polygamma(1)
        da, db = a - q1, b - q2
        return 0.5 * ((ta + tab) * da ** 2 + 2 * tab * da * db + (tb + tab) * db ** 2).sum(-1)
    raise KeyError(kind)


@pytest.mark.parametrize("kind", list(orc.KINDS))
@pytest.mark.parametrize("layout", LAYOUTS)
def test_backward_matches_autograd(kind, layout):
    be, ne, bc, nc = layout
    rng = np.random.default_rng(_seed("b", kind, layout))
    e, q1, q2 = make_inputs(kind, be, ne, bc, nc, 9, rng)
    bsize, num = max(be, bc), max(ne, nc)
    gout = rng.standard_normal((bsize, num))
    te = torch.tensor(e, requires_grad=True)
    t1 = torch.tensor(q1, requires_grad=True)
    t2 = None if q2 is None else torch.tensor(q2, requires_grad=True)
    ii, jj = torch.meshgrid(torch.arange(bsize), torch.arange(num), indexing="ij")
    out = torch_form(kind, te[ii % be, jj % ne], t1[ii % bc, jj % nc], None if t2 is None else t2[ii % bc, jj % nc])
    (out * torch.from_numpy(gout)).sum().backward()
    gent, gq1, gq2 = orc.dist_backward(kind, gout, e, q1, q2)
    tol = 3e-7 if kind.startswith("beta") else 1e-10
    assert np.allclose(gent, te.grad.numpy(), rtol=tol, atol=tol)
    assert np.allclose(gq1, t1.grad.numpy(), rtol=tol, atol=tol)
    if q2 is not None:
        assert np.allclose(gq2, t2.grad.numpy(), rtol=tol, atol=tol)


@pytest.mark.parametrize("kind", ["l2", "rotate", "beta_kl", "box_out", "box_in"])
def test_backward_matches_finite_differences(kind):
    rng = np.random.default_rng(11)
    e, q1, q2 = make_inputs(kind, 3, 2, 3, 1, 5, rng, positive=True)
    gout = rng.standard_normal((3, 2))
    gent, gq1, gq2 = orc.dist_backward(kind, gout, e, q1, q2)
    h = 1e-6

    def loss(e_, a_, b_):
        return float((orc.dist_forward(kind, e_, a_, b_) * gout).sum())

    for arr, grad in ((e, gent), (q1, gq1), (q2, gq2)):
        if arr is None:
            continue
        flat = arr.reshape(-1)
        for k in rng.choice(flat.size, size=min(12, flat.size), replace=False):
            old = flat[k]
            flat[k] = old + h
            up = loss(e, q1, q2)
            flat[k] = old - h
            dn = loss(e, q1, q2)
            flat[k] = old
            assert abs((up - dn) / (2 * h) - grad.reshape(-1)[k]) < 2e-5


def test_tie_conventions_follow_the_kernel():
    one = lambda *v: np.array(v, dtype=np.float64).reshape(1, 1, -1)
    g = np.array([[2.0]])
    # l1 at e == c: sign(0) = -1
    gent, gq, _ = orc.dist_backward("l1", g, one(0.5), one(0.5))
    assert gent.item() == -2.0 and gq.item() == 2.0
    # box_out at |e-c| - o == 0 passes gradient (>=); e-c = 0.25 > 0
    gent, gc, go = orc.dist_backward("box_out", g, one(1.0), one(0.75), one(0.25))
    assert (gent.item(), gc.item(), go.item()) == (2.0, -2.0, -2.0)
    # box_out inside the box: no gradient at all
    gent, gc, go = orc.dist_backward("box_out", g, one(1.0), one(0.75), one(0.5))
    assert (gent.item(), gc.item(), go.item()) == (0.0, 0.0, 0.0)
    # box_out with e == c and o == 0: relu argument is 0 -> passes, sign(0) = -1
    gent, gc, go = orc.dist_backward("box_out", g, one(1.0), one(1.0), one(0.0))
    assert (gent.item(), gc.item(), go.item()) == (-2.0, 2.0, -2.0)
    # box_in tie |e-c| == o goes to the offset branch
    gent, gc, go = orc.dist_backward("box_in", g, one(1.0), one(0.75), one(0.25))
    assert (gent.item(), gc.item(), go.item()) == (0.0, 0.0, 2.0)
    # box_in inside: gradient to entity / center with inner sign
    gent, gc, go = orc.dist_backward("box_in", g, one(0.5), one(0.75), one(0.5))
    assert (gent.item(), gc.item(), go.item()) == (-2.0, 2.0, 0.0)
    # box_in with negative offset: min(...) <= 0 -> outer sign -1, offset branch
    gent, gc, go = orc.dist_backward("box_in", g, one(1.0), one(0.75), one(-0.5))
    assert (gent.item(), gc.item(), go.item()) == (0.0, 0.0, -2.0)
    assert orc.dist_forward("box_in", one(1.0), one(0.75), one(-0.5)).item() == 0.5
    # box_in with e == c (min = 0 -> outer sign -1, inner sign(0) = -1)
    gent, gc, go = orc.dist_backward("box_in", g, one(1.0), one(1.0), one(0.5))
    assert (gent.item(), gc.item(), go.item()) == (2.0, -2.0, 0.0)
    # rotate at zero distance: eps inside the root keeps everything finite and zero
    gent, gr, gi = orc.dist_backward("rotate", g, one(0.3, 0.4), one(0.3), one(0.4))
    assert np.all(gent == 0) and gr.item() == 0 and gi.item() == 0
    assert abs(orc.dist_forward("rotate", one(0.3, 0.4), one(0.3), one(0.4)).item() - 1e-10) < 1e-16


# ---------------------------------------------------------------- gather / merge / Adam

def test_gather_and_regularizer():
    t = RNG.standard_normal((50, 6))
    idx = RNG.integers(0, 50, size=(7, 5))
    assert np.array_equal(orc.gather(t, idx), t[idx.reshape(-1)])
    with pytest.raises(IndexError):
        orc.gather(t, np.array([50]))
    with pytest.raises(IndexError):
        orc.gather(t, np.array([-1]))
    x = RNG.standard_normal(100) * 3
    assert np.array_equal(orc.regularizer(x), np.clip(x + 1, 0.05, 1e9))


@pytest.mark.parametrize("p,n", [(1, 5), (64, 4), (1000, 50), (1000, 10 ** 9), (17, 1)])
def test_merge_indices_is_numpy_unique(p, n):
    idx = RNG.integers(0, n, size=p)
    uniq, inverse, order, seg = orc.merge_indices(idx)
    u2, inv2 = np.unique(idx, return_inverse=True)
    assert np.array_equal(uniq, u2) and np.array_equal(inverse, inv2)
    assert np.array_equal(order, np.argsort(idx, kind="stable"))
    assert seg[0] == 0 and seg[-1] == p and np.all(np.diff(seg) > 0)
    assert np.array_equal(np.diff(seg), np.bincount(inv2))
    assert np.all(np.diff(uniq) > 0)


def test_merge_indices_empty():
    uniq, inverse, order, seg = orc.merge_indices(np.zeros(0, dtype=np.int64))
    assert uniq.size == 0 and seg.tolist() == [0]


def test_merge_grads_is_add_at():
    idx = RNG.integers(0, 30, size=400)
    g = RNG.standard_normal((400, 7))
    uniq, inverse, _, _ = orc.merge_indices(idx)
    want = np.zeros((uniq.size, 7))
    np.add.at(want, inverse, g)
    assert np.allclose(orc.merge_grads(g, inverse, uniq.size), want, rtol=1e-13, atol=1e-13)


def test_adam_equals_torch_adam_when_every_row_is_touched():
    n, d, lr = 12, 5, 1e-2
    w0 = RNG.standard_normal((n, d))
    w, m, v = w0.copy(), np.zeros((n, d)), np.zeros((n, d))
    tw = torch.tensor(w0.copy(), requires_grad=True)
    opt = torch.optim.Adam([tw], lr=lr, betas=(0.9, 0.999), eps=1e-8)
    for step in range(1, 6):
        g = RNG.standard_normal((n, d))
        perm = RNG.permutation(n)
        orc.adam_rows(w, m, v, np.sort(perm), g, lr, step)
        tw.grad = torch.tensor(g)
        opt.step()
        assert np.allclose(w, tw.detach().numpy(), rtol=1e-12, atol=1e-12)
    st = opt.state[tw]
    assert np.allclose(m, st["exp_avg"].numpy(), rtol=1e-12)
    assert np.allclose(v, st["exp_avg_sq"].numpy(), rtol=1e-12)


def test_adam_is_lazy_and_uses_the_global_step():
    n, d, lr = 10, 4, 1e-3
    w = RNG.standard_normal((n, d))
    m, v = np.zeros((n, d)), np.zeros((n, d))
    w0 = w.copy()
    g = RNG.standard_normal((2, d))
    # first touch happens at global step 3: bias correction uses t = 3, not 1
    orc.adam_rows(w, m, v, np.array([2, 7]), g, lr, step=3)
    untouched = [r for r in range(n) if r not in (2, 7)]
    assert np.array_equal(w[untouched], w0[untouched])
    assert not m[untouched].any() and not v[untouched].any()
    m1, v1 = 0.1 * g, 0.001 * g * g
    denom = np.sqrt(v1) / math.sqrt(1 - 0.999 ** 3) + 1e-8
    want = w0[[2, 7]] - lr / (1 - 0.9 ** 3) * m1 / denom
    assert np.allclose(w[[2, 7]], want, rtol=1e-13)
    assert np.allclose(m[[2, 7]], m1, rtol=1e-13) and np.allclose(v[[2, 7]], v1, rtol=1e-13)
    # a touched row with an exactly zero gradient still moves by momentum
    wb = w.copy()
    orc.adam_rows(w, m, v, np.array([2]), np.zeros((1, d)), lr, step=4)
    assert np.all(w[2] != wb[2]) and np.array_equal(w[7], wb[7])


def test_adam_squeeze_variant_closed_form():
    n, d, lr = 6, 8, 1e-3
    w = RNG.standard_normal((n, d))
    m, v = np.zeros((n, d)), np.full((n, 1), 0.25)
    w0 = w.copy()
    g = RNG.standard_normal((1, d))
    orc.adam_rows(w, m, v, np.array([4]), g, lr, step=2, squeeze=True)
    v1 = 0.999 * 0.25 + 0.001 * np.mean(g * g)
    assert abs(v[4, 0] - v1) < 1e-15 and np.all(v[[0, 1, 2, 3, 5]] == 0.25)
    want = w0[4] - lr / (1 - 0.9 ** 2) * (0.1 * g[0]) / (math.sqrt(v1) / math.sqrt(1 - 0.999 ** 2) + 1e-8)
    assert np.allclose(w[4], want, rtol=1e-13)


@pytest.mark.parametrize("name", ["sgd", "adagrad", "rmsprop"])
def test_other_row_optimizers_equal_torch_when_every_row_is_touched(name):
    n, d, lr = 9, 5, 1e-2
    w0 = RNG.standard_normal((n, d))
    w, state = w0.copy(), np.zeros((n, d))
    tw = torch.tensor(w0.copy(), requires_grad=True)
    opt = {"sgd": lambda: torch.optim.SGD([tw], lr=lr),
           "adagrad": lambda: torch.optim.Adagrad([tw], lr=lr, eps=1e-8),
           "rmsprop": lambda: torch.optim.RMSprop([tw], lr=lr, alpha=0.99, eps=1e-8)}[name]()
    for _ in range(4):
        g = RNG.standard_normal((n, d))
        if name == "sgd":
            orc.sgd_rows(w, np.arange(n), g, lr)
        elif name == "adagrad":
            orc.adagrad_rows(w, state, np.arange(n), g, lr)
        else:
            orc.rmsprop_rows(w, state, np.arange(n), g, lr)
        tw.grad = torch.tensor(g)
        opt.step()
        assert np.allclose(w, tw.detach().numpy(), rtol=1e-12, atol=1e-12)


def test_other_row_optimizers_are_lazy_and_squeeze_by_closed_form():
    n, d, lr = 7, 6, 1e-2
    w0 = RNG.standard_normal((n, d))
    g = RNG.standard_normal((2, d))
    rows = np.array([1, 4])
    gm = (g * g).mean(1, keepdims=True)
    w, st = w0.copy(), np.full((n, 1), 0.5)
    orc.adagrad_rows(w, st, rows, g, lr, squeeze=True)
    assert np.allclose(st[rows], 0.5 + gm, rtol=1e-14) and np.all(st[[0, 2, 3, 5, 6]] == 0.5)
    assert np.allclose(w[rows], w0[rows] - lr * g / (np.sqrt(0.5 + gm) + 1e-8), rtol=1e-13)
    assert np.array_equal(w[[0, 2, 3, 5, 6]], w0[[0, 2, 3, 5, 6]])
    w, st = w0.copy(), np.full((n, 1), 0.5)
    orc.rmsprop_rows(w, st, rows, g, lr, squeeze=True)
    s1 = 0.99 * 0.5 + 0.01 * gm
    assert np.allclose(st[rows], s1, rtol=1e-14)
    assert np.allclose(w[rows], w0[rows] - lr * g / (np.sqrt(s1) + 1e-8), rtol=1e-13)


# ---------------------------------------------------------------- composition

def test_scores_match_native_cal_logit_forms():
    rng = np.random.default_rng(5)
    b, k, d = 4, 6, 10
    rows = rng.standard_normal((b, k, d))
    c, o = rng.standard_normal((b, 1, d)), np.abs(rng.standard_normal((b, 1, d)))
    delta = np.abs(rows - c)
    want = 24 - np.maximum(delta - o, 0).sum(-1) - 0.02 * np.minimum(delta, o).sum(-1)
    assert np.allclose(orc.score_forward("box", rows, c, o, 24.0, 0.02), want, rtol=1e-12)
    assert np.allclose(orc.score_forward("l2", rows, c, None, 12.0), 12 - np.linalg.norm(rows - c, axis=-1), rtol=1e-12)
    assert np.allclose(orc.score_forward("l1", rows, c, None, 12.0), 12 - np.abs(rows - c).sum(-1), rtol=1e-12)
    rows2 = rng.standard_normal((b, k, 2 * d))
    re, im = rng.standard_normal((b, 1, d)), rng.standard_normal((b, 1, d))
    want = 9 - np.sqrt((rows2[..., :d] - re) ** 2 + (rows2[..., d:] - im) ** 2).sum(-1)
    assert np.allclose(orc.score_forward("rotate", rows2, re, im, 9.0), want, rtol=1e-12)


def test_score_backward_matches_autograd_l2_and_box():
    rng = np.random.default_rng(6)
    b, k, d = 3, 5, 7
    rows = rng.standard_normal((b, k, d))
    c, o = rng.standard_normal((b, 1, d)), np.abs(rng.standard_normal((b, 1, d)))
    gs = rng.standard_normal((b, k))
    tr, tc, to = (torch.tensor(x, requires_grad=True) for x in (rows, c, o))
    s = 12 - torch.linalg.norm(tr - tc, dim=-1)
    (s * torch.from_numpy(gs)).sum().backward()
    gr, gc, _ = orc.score_backward("l2", gs, rows, c)
    assert np.allclose(gr, tr.grad.numpy(), rtol=1e-11) and np.allclose(gc, tc.grad.numpy(), rtol=1e-11)
    tr.grad = tc.grad = None
    delta = (tr - tc).abs()
    s = 24 - torch.relu(delta - to).sum(-1) - 0.02 * torch.minimum(delta, to).sum(-1)
    (s * torch.from_numpy(gs)).sum().backward()
    gr, gc, go = orc.score_backward("box", gs, rows, c, o, cen=0.02)
    assert np.allclose(gr, tr.grad.numpy(), rtol=1e-11, atol=1e-14)
    assert np.allclose(gc, tc.grad.numpy(), rtol=1e-11, atol=1e-14)
    assert np.allclose(go, to.grad.numpy(), rtol=1e-11, atol=1e-14)


def test_similarity_and_two_half_scores_match_autograd_of_the_closed_forms():
    """score_forward / score_backward for the models the two tests above leave open: ComplEx and DistMult, whose
    logit is gamma + similarity (models/complex.py:140-148; naive_complex_sim, complex_dist.py:67-70;
    naive_innerprod, distmult_dist.py:66-68) -- a flipped sign on the coefficient would pass every distance
    test -- RotatE (naive_rotate_dist, rotate_dist.py:68-75) and Beta-KL (torch.distributions' _kl_beta_beta,
    beta.py:298)."""
    rng = np.random.default_rng(16)
    b, k, d = 3, 5, 6
    gs = rng.standard_normal((b, k))
    t = lambda x: torch.tensor(x, requires_grad=True)

    def check(model, rows, q1, q2, gamma, closed_form):
        tr, t1 = t(rows), t(q1)
        t2 = None if q2 is None else t(q2)
        s = closed_form(tr, t1, t2)
        assert np.allclose(orc.score_forward(model, rows, q1, q2, gamma), s.detach().numpy(), rtol=1e-11, atol=1e-13), model
        (s * torch.from_numpy(gs)).sum().backward()
        gr, g1, g2 = orc.score_backward(model, gs, rows, q1, q2)
        assert np.allclose(gr, tr.grad.numpy(), rtol=1e-9, atol=1e-12), model
        assert np.allclose(g1, t1.grad.numpy(), rtol=1e-9, atol=1e-12), model
        if q2 is not None:
            assert np.allclose(g2, t2.grad.numpy(), rtol=1e-9, atol=1e-12), model

    rows2 = rng.standard_normal((b, k, 2 * d))
    re, im = rng.standard_normal((b, 1, d)), rng.standard_normal((b, 1, d))
    check("complex", rows2, re, im, 3.0, lambda e, a, c: 3.0 + (e[..., :d] * a + e[..., d:] * c).sum(-1))
    check("rotate", rows2, re, im, 9.0,
          lambda e, a, c: 9.0 - torch.sqrt((e[..., :d] - a) ** 2 + (e[..., d:] - c) ** 2).sum(-1))
    rows1, q = rng.standard_normal((b, k, d)), rng.standard_normal((b, 1, d))
    check("distmult", rows1, q, None, 2.0, lambda e, a, c: 2.0 + (e * a).sum(-1))
    pos = lambda *sh: np.clip(1 + rng.standard_normal(sh), 0.05, 1e9)
    rows_b, qa, qb = pos(b, k, 2 * d), pos(b, 1, d), pos(b, 1, d)
    kl = torch.distributions.kl._kl_beta_beta
    check("beta_kl", rows_b, qa, qb, 60.0,
          lambda e, a, c: 60.0 - kl(torch.distributions.Beta(e[..., :d], e[..., d:]), torch.distributions.Beta(a, c)).sum(-1))


def test_unit_halves_is_f_normalize_per_half_and_its_backward_is_autograd():
    """unit_halves / unit_halves_backward and the `norm` form of the ComplEx score (models/complex.py:142-146 with
    embed_norm = F.normalize, common/modules.py:38-40).  torch's own normalize is the routine the reference calls;
    the properties below catch what a comparison of two implementations of the same formula would not: a result
    that is not of unit length, a gradient with a component along the row (the dropped projection term), a
    wrong power of the length (finite differences)."""
    rng = np.random.default_rng(31)
    b, k, d = 3, 4, 5
    rows = rng.standard_normal((b, k, 2 * d)) * rng.uniform(0.1, 5.0, (b, k, 1))
    un = orc.unit_halves(rows)
    assert np.allclose((un[..., :d] ** 2).sum(-1), 1.0, atol=1e-14) and np.allclose((un[..., d:] ** 2).sum(-1), 1.0, atol=1e-14)
    tr = torch.tensor(rows, requires_grad=True)
    F = torch.nn.functional
    tn = torch.cat((F.normalize(tr[..., :d], p=2, dim=-1), F.normalize(tr[..., d:], p=2, dim=-1)), dim=-1)
    assert np.allclose(un, tn.detach().numpy(), rtol=1e-14, atol=0)
    g = rng.standard_normal(rows.shape)
    (tn * torch.from_numpy(g)).sum().backward()
    gb = orc.unit_halves_backward(rows, g)
    assert np.allclose(gb, tr.grad.numpy(), rtol=1e-11, atol=1e-13)
    # scaling a row does not change the result: the gradient has no component along it
    assert np.abs((gb[..., :d] * rows[..., :d]).sum(-1)).max() < 1e-12
    assert np.abs((gb[..., d:] * rows[..., d:]).sum(-1)).max() < 1e-12
    # central finite differences of sum(g * unit_halves(rows))
    f = lambda x: (g * orc.unit_halves(x)).sum()
    h = 1e-6
    for pos in [(0, 0, 0), (1, 2, d - 1), (2, 3, d), (0, 1, 2 * d - 1)]:
        hi, lo = rows.copy(), rows.copy()
        hi[pos] += h
        lo[pos] -= h
        assert abs((f(hi) - f(lo)) / (2 * h) - gb[pos]) < 1e-7 * max(1.0, abs(gb[pos]))
    # a half shorter than eps is divided by eps, and so is its gradient (the clamp's constant branch)
    tiny = np.zeros((1, 1, 4))
    tiny[0, 0, :2] = [3e-13, 4e-13]          # length 5e-13 < 1e-12
    tiny[0, 0, 2:] = [3.0, 4.0]
    assert np.allclose(orc.unit_halves(tiny)[0, 0], [0.3, 0.4, 0.6, 0.8], rtol=1e-12)
    gt = orc.unit_halves_backward(tiny, np.ones((1, 1, 4)))[0, 0]
    assert np.allclose(gt[:2], [1e12, 1e12]) and np.allclose(gt[2:], [(1 - 0.6 * 1.4) / 5, (1 - 0.8 * 1.4) / 5], rtol=1e-12)
    # one half = the whole row (DistMult's 'norm' mode, distmult.py:129-130): F.normalize of the row and its autograd
    tw = torch.tensor(rows, requires_grad=True)
    whole = F.normalize(tw, p=2, dim=-1)
    assert np.allclose(orc.unit_halves(rows, halves=1), whole.detach().numpy(), rtol=1e-14, atol=0)
    (whole * torch.from_numpy(g)).sum().backward()
    assert np.allclose(orc.unit_halves_backward(rows, g, halves=1), tw.grad.numpy(), rtol=1e-11, atol=1e-13)
    qd = rng.standard_normal((b, 1, 2 * d))
    td = torch.tensor(qd, requires_grad=True)
    tw.grad = None
    sd = (F.normalize(tw, p=2, dim=-1) * td).sum(-1)
    gsd = rng.standard_normal((b, k))
    assert np.allclose(orc.score_forward("distmult", rows, qd, None, 0.0, norm=True), sd.detach().numpy(), rtol=1e-12, atol=1e-14)
    (sd * torch.from_numpy(gsd)).sum().backward()
    grd, gqd, _ = orc.score_backward("distmult", gsd, rows, qd, None, norm=True)
    assert np.allclose(grd, tw.grad.numpy(), rtol=1e-10, atol=1e-13) and np.allclose(gqd, td.grad.numpy(), rtol=1e-10, atol=1e-13)
    # the ComplEx logit over the scaled rows, and its three gradients, against autograd of the model's lines
    re, im = rng.standard_normal((b, 1, d)), rng.standard_normal((b, 1, d))
    gs = rng.standard_normal((b, k))
    tr = torch.tensor(rows, requires_grad=True)
    t1, t2 = torch.tensor(re, requires_grad=True), torch.tensor(im, requires_grad=True)
    e_re, e_im = torch.chunk(tr, 2, dim=-1)
    ent = torch.cat((F.normalize(e_re, p=2, dim=-1), F.normalize(e_im, p=2, dim=-1)), dim=-1)
    s = 0.5 + (ent[..., :d] * t1 + ent[..., d:] * t2).sum(-1)
    assert np.allclose(orc.score_forward("complex", rows, re, im, 0.5, norm=True), s.detach().numpy(), rtol=1e-12, atol=1e-14)
    (s * torch.from_numpy(gs)).sum().backward()
    gr, g1, g2 = orc.score_backward("complex", gs, rows, re, im, norm=True)
    assert np.allclose(gr, tr.grad.numpy(), rtol=1e-10, atol=1e-13)
    assert np.allclose(g1, t1.grad.numpy(), rtol=1e-10, atol=1e-13)
    assert np.allclose(g2, t2.grad.numpy(), rtol=1e-10, atol=1e-13)


def test_train_step_equals_dense_autograd_pipeline():
    """gather -> score -> backward -> merge -> Adam equals autograd through table[idx]
    followed by a dense Adam restricted to the touched rows."""
    rng = np.random.default_rng(8)
    n, d, b, k = 40, 6, 5, 9
    table = rng.uniform(-0.07, 0.07, (n, d))
    m, v = np.zeros((n, d)), np.zeros((n, d))
    c, o = rng.uniform(-0.07, 0.07, (b, 1, d)), np.abs(rng.uniform(-0.07, 0.07, (b, 1, d)))
    idx = rng.integers(0, n, (b, k))
    gs = rng.standard_normal((b, k))
    tt = torch.tensor(table.copy(), requires_grad=True)
    rows = tt[torch.from_numpy(idx)]
    delta = (rows - torch.from_numpy(c)).abs()
    s = 24 - torch.relu(delta - torch.from_numpy(o)).sum(-1) - 0.02 * torch.minimum(delta, torch.from_numpy(o)).sum(-1)
    (s * torch.from_numpy(gs)).sum().backward()
    t0 = table.copy()
    res = orc.train_step("box", table, m, v, idx, c, o, gs, 24.0, 0.02, 1e-4, 1)
    assert np.allclose(res["score"], s.detach().numpy(), rtol=1e-12)
    dense = np.zeros((n, d))
    dense[res["uniq"]] = res["merged"]
    assert np.allclose(dense, tt.grad.numpy(), rtol=1e-11, atol=1e-14)
    touched = np.zeros(n, bool)
    touched[idx.reshape(-1)] = True
    assert np.array_equal(np.flatnonzero(touched), res["uniq"])
    assert np.array_equal(table[~touched], t0[~touched])
    g = tt.grad.numpy()[touched]
    want = t0[touched] - 1e-4 / 0.1 * (0.1 * g) / (np.sqrt(0.001 * g * g) / math.sqrt(0.001) + 1e-8)
    assert np.allclose(table[touched], want, rtol=1e-11)


@pytest.mark.parametrize("temperature", [0.0, 0.7])
@pytest.mark.parametrize("weighted", [False, True])
@pytest.mark.parametrize("masked", [False, True])
def test_sample_loss_is_the_torch_expression_of_the_training_step(temperature, weighted, masked):
    """orc.sample_loss against torch autograd of the expression as train_process.py:194-213 writes it
    (F.softmax(...).detach() * F.logsigmoid(-x), weighted or plain means, / 2 / world_size)."""
    import torch.nn.functional as F
    rng = np.random.default_rng(17)
    b, k, world = 6, 11, 4
    pos, neg = rng.standard_normal(b) * 4, rng.standard_normal((b, k)) * 4
    neg[0, 0], pos[1] = 60.0, -70.0                      # saturated sigmoids
    mask = (rng.random((b, k)) > 0.3).astype(np.float64)
    w = rng.random(b) + 0.1
    tp, tn = torch.tensor(pos, requires_grad=True), torch.tensor(neg, requires_grad=True)
    x = tn * torch.tensor(mask) if masked else tn
    if temperature > 0:
        s = (F.softmax(x * temperature, dim=1).detach() * F.logsigmoid(-x)).sum(dim=1)
    else:
        s = F.logsigmoid(-x).mean(dim=1)
    p = F.logsigmoid(tp)
    if weighted:
        tw = torch.tensor(w)
        pl, nl = -(tw * p).sum() / tw.sum(), -(tw * s).sum() / tw.sum()
    else:
        pl, nl = -p.mean(), -s.mean()
    ((pl + nl) / 2 / world).backward()
    got = orc.sample_loss(pos, neg, mask if masked else None, w if weighted else None, temperature, 0.5 / world)
    assert abs(got[0] - pl.item()) < 1e-12 and abs(got[1] - nl.item()) < 1e-12
    assert np.allclose(got[2], tp.grad.numpy(), rtol=1e-12, atol=1e-15)
    assert np.allclose(got[3], tn.grad.numpy(), rtol=1e-12, atol=1e-15)


def test_sample_loss_known_values():
    """All logits 0: logsigmoid(0) = -ln 2, sigmoid(0) = 1/2, softmax uniform."""
    b, k = 3, 5
    for t in (0.0, 2.0):
        pl, nl, gp, gn = orc.sample_loss(np.zeros(b), np.zeros((b, k)), temperature=t, scale=0.5)
        assert abs(pl - math.log(2)) < 1e-15 and abs(nl - math.log(2)) < 1e-15
        assert np.allclose(gp, -0.5 / b * 0.5) and np.allclose(gn, 0.5 / b / k * 0.5)


def test_filtered_ranks_follow_the_evaluation_loop():
    """orc.filtered_ranks against (1) the tensor recipe of train_process.py:124-145 restated with torch
    (argsort, scatter of arange, sort of the answers' ranks, minus arange, +1, hard mask) on tie-free
    scores, and (2) the definition 1 + #non-answers with a larger score."""
    rng = np.random.default_rng(23)
    n = 400
    scores = rng.permutation(n).astype(np.float64) * 0.37 - 20     # tie-free
    easy, hard = [5, 17, 300, 42], [7, 399, 0, 123, 250]
    got_h, got_e = orc.filtered_ranks(scores, easy, hard)
    logit = torch.tensor(scores)[None]
    argsort = torch.argsort(logit, dim=1, descending=True)
    ranking = argsort.clone().to(torch.float)
    ranking = ranking.scatter_(1, argsort, torch.arange(n).to(torch.float).repeat(1, 1))
    cur = ranking[0, easy + hard]
    cur, indices = torch.sort(cur)
    masks = indices >= len(easy)
    cur = cur - torch.arange(len(easy) + len(hard)).to(torch.float) + 1
    assert sorted(got_h.tolist()) == cur[masks].to(torch.int64).tolist()
    is_ans = np.zeros(n, bool)
    is_ans[easy + hard] = True
    for a, r in zip(hard + easy, list(got_h) + list(got_e)):
        assert r == 1 + int(((scores > scores[a]) & ~is_ans).sum())
    # equal logits: the lower id ranks first
    tied = np.zeros(6)
    h, e = orc.filtered_ranks(tied, [], [4])
    assert h.tolist() == [5] and e.size == 0
    h, _ = orc.filtered_ranks(tied, [1], [4, 0])
    assert h.tolist() == [3, 1]      # position 4, two answers (ids 0 and 1) before it


def test_candidate_ranks_follow_the_sampled_negatives_branch():
    """orc.candidate_ranks against the tensor recipe of train_process.py:118-128, 141-147 restated with torch
    (where / bias, argsort, scatter of arange, ranking[:num_hard], sort, minus arange, +1) on tie-free logits, and
    the tie rule by hand."""
    rng = np.random.default_rng(29)
    c, n_hard = 300, 6
    neg = rng.integers(0, 1000, c)
    neg[[40, 41, 299]] = -1
    logit = (rng.permutation(c).astype(np.float32) * np.float32(0.37) - np.float32(20.0))
    biased, ranking, filt = orc.candidate_ranks(logit, neg, n_hard)
    t_neg = torch.tensor(neg)[None]
    bias = torch.where(t_neg == -1, -1e6, 0.)
    negative_logit = torch.tensor(logit)[None] + bias.to(torch.float32)
    assert np.array_equal(biased, negative_logit[0].numpy())
    argsort = torch.argsort(negative_logit, dim=1, descending=True)
    rk = argsort.clone().to(torch.float)
    rk = rk.scatter_(1, argsort, torch.arange(c).to(torch.float).repeat(1, 1))
    assert np.array_equal(ranking, rk[0].to(torch.int64).numpy())
    cur, _ = torch.sort(rk[0, :n_hard])
    cur = cur - torch.arange(n_hard).to(torch.float) + 1
    assert sorted(filt.tolist()) == cur.to(torch.int64).tolist()
    assert ranking[40] > ranking[(neg != -1)].max() and ranking[41] == ranking[40] + 1    # padding last, in position order
    # equal logits: the lower position first
    _, r, f = orc.candidate_ranks(np.zeros(5, np.float32), np.array([3, 3, -1, 3, 3]), 2)
    assert r.tolist() == [0, 1, 4, 2, 3] and f.tolist() == [1, 1]
