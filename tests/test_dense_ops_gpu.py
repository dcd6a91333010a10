"""HIP dense distance operators against the CPU oracle, through the extlib_cuda-shaped
surface (smore_amd.extlib_hip -> C ABI) and through the autograd operators."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests.util import REL_F32, REL_F64, assert_close, make_inputs, seed

pytestmark = pytest.mark.gpu

LAYOUTS = [
    (6, 5, 6, 1),    # per-query negatives
    (1, 7, 4, 1),    # shared negatives
    (5, 1, 5, 1),    # positives
    (1, 33, 1, 1),   # eval against all entities
    (4, 1, 4, 6),    # reverse queries
    (30, 1, 1, 20),  # the reference's smoke-test layout
    (6, 4, 3, 2),    # both sides broadcast by modulo
]
DIMS = [1, 7, 64, 200]


def _dev(a, dtype):
    return None if a is None else torch.tensor(a, dtype=dtype, device="cuda")


@pytest.mark.parametrize("kind", list(orc.KINDS))
@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_dense_forward_backward(kind, layout, dtype):
    from smore_amd import extlib_hip as ext
    be, ne, bc, nc = layout
    for dim in DIMS:
        rng = np.random.default_rng(seed(kind, layout, dim))
        e, q1, q2 = make_inputs(kind, be, ne, bc, nc, dim, rng)
        bsize, num = max(be, bc), max(ne, nc)
        gout = rng.standard_normal((bsize, num))
        if dtype == torch.float32:  # the oracle sees exactly the fp32 values the device sees
            e, q1, gout = (x.astype(np.float32).astype(np.float64) for x in (e, q1, gout))
            q2 = None if q2 is None else q2.astype(np.float32).astype(np.float64)
        te, t1, t2, tg = _dev(e, dtype), _dev(q1, dtype), _dev(q2, dtype), _dev(gout, dtype)
        dst = torch.full((bsize, num), float("nan"), dtype=dtype, device="cuda")
        ext.dist_forward(kind, te, t1, t2, dst, t2 is not None)
        rel = REL_F32 if dtype == torch.float32 else REL_F64
        if dtype == torch.float64 and kind.startswith("beta"):
            rel = 1e-9
        assert_close(dst.cpu().numpy(), orc.dist_forward(kind, e, q1, q2), rel, f"{kind} fwd dim={dim}")
        ge = torch.full_like(te, float("nan"))
        g1 = torch.full_like(t1, float("nan"))
        g2 = None if t2 is None else torch.full_like(t2, float("nan"))
        ext.dist_backward(kind, tg, te, t1, t2, ge, g1, g2, t2 is not None)
        oe, o1, o2 = orc.dist_backward(kind, gout, e, q1, q2)
        assert_close(ge.cpu().numpy(), oe, rel, f"{kind} gent dim={dim}")
        assert_close(g1.cpu().numpy(), o1, rel, f"{kind} gq1 dim={dim}")
        if t2 is not None:
            assert_close(g2.cpu().numpy(), o2, rel, f"{kind} gq2 dim={dim}")


@pytest.mark.parametrize("kind", list(orc.KINDS))
@pytest.mark.parametrize("layout", [(6, 9, 6, 1), (1, 11, 5, 1), (4, 1, 4, 1), (5, 1, 5, 10)])
def test_long_rows_in_the_per_query_and_shared_layouts(kind, layout):
    """Rows of two and four 256-float column groups (and one just past the vector kernels' 1024-float limit)
    in the layouts that have their own fp32 kernels: per-query negatives, shared negatives, positives, reverse."""
    from smore_amd import extlib_hip as ext
    be, ne, bc, nc = layout
    for dim in (260, 400, 516, 1000, 1024, 1028):
        rng = np.random.default_rng(seed(kind, layout, dim))
        e, q1, q2 = make_inputs(kind, be, ne, bc, nc, dim, rng)
        bsize, num = max(be, bc), max(ne, nc)
        gout = rng.standard_normal((bsize, num))
        e, q1, gout = (x.astype(np.float32).astype(np.float64) for x in (e, q1, gout))
        q2 = None if q2 is None else q2.astype(np.float32).astype(np.float64)
        te, t1, t2, tg = (_dev(x, torch.float32) for x in (e, q1, q2, gout))
        dst = torch.full((bsize, num), float("nan"), device="cuda")
        ext.dist_forward(kind, te, t1, t2, dst, t2 is not None)
        assert_close(dst.cpu().numpy(), orc.dist_forward(kind, e, q1, q2), REL_F32, f"{kind} fwd dim={dim}")
        ge, g1 = torch.full_like(te, float("nan")), torch.full_like(t1, float("nan"))
        g2 = None if t2 is None else torch.full_like(t2, float("nan"))
        ext.dist_backward(kind, tg, te, t1, t2, ge, g1, g2, t2 is not None)
        oe, o1, o2 = orc.dist_backward(kind, gout, e, q1, q2)
        assert_close(ge.cpu().numpy(), oe, REL_F32, f"{kind} gent dim={dim}")
        assert_close(g1.cpu().numpy(), o1, REL_F32, f"{kind} gq1 dim={dim}")
        if t2 is not None:
            assert_close(g2.cpu().numpy(), o2, REL_F32, f"{kind} gq2 dim={dim}")


def _random_layouts(count=48):
    """Seeded random broadcast layouts (each axis equal, or one side a multiple of the other), dims on and
    off the 16-byte path, both precisions: exercises the choice between the layout-specific and the general
    kernels."""
    rng = np.random.default_rng(77)
    kinds = list(orc.KINDS)
    cases = []
    for i in range(count):
        def pair():
            a, m = int(rng.choice([1, 2, 3, 5, 8, 33])), int(rng.choice([1, 1, 2, 3]))
            return (a, a * m) if rng.random() < 0.5 else (a * m, a)
        (be, bc), (ne, nc) = pair(), pair()
        dim = int(rng.choice([1, 3, 4, 16, 63, 64, 200, 257, 400, 1000]))
        cases.append((kinds[i % len(kinds)], be, ne, bc, nc, dim, "f32" if i % 3 else "f64"))
    return cases


@pytest.mark.parametrize("case", _random_layouts(), ids=lambda c: "-".join(str(x) for x in c))
def test_random_broadcast_layouts(case):
    from smore_amd import extlib_hip as ext
    kind, be, ne, bc, nc, dim, prec = case
    dtype = torch.float32 if prec == "f32" else torch.float64
    rng = np.random.default_rng(seed(*case))
    e, q1, q2 = make_inputs(kind, be, ne, bc, nc, dim, rng)
    bsize, num = max(be, bc), max(ne, nc)
    gout = rng.standard_normal((bsize, num))
    if dtype == torch.float32:
        e, q1, gout = (x.astype(np.float32).astype(np.float64) for x in (e, q1, gout))
        q2 = None if q2 is None else q2.astype(np.float32).astype(np.float64)
    te, t1, t2, tg = (_dev(x, dtype) for x in (e, q1, q2, gout))
    rel = REL_F32 if dtype == torch.float32 else (1e-9 if kind.startswith("beta") else REL_F64)
    dst = torch.full((bsize, num), float("nan"), dtype=dtype, device="cuda")
    ext.dist_forward(kind, te, t1, t2, dst, t2 is not None)
    assert_close(dst.cpu().numpy(), orc.dist_forward(kind, e, q1, q2), rel, "forward")
    ge, g1 = torch.full_like(te, float("nan")), torch.full_like(t1, float("nan"))
    g2 = None if t2 is None else torch.full_like(t2, float("nan"))
    ext.dist_backward(kind, tg, te, t1, t2, ge, g1, g2, t2 is not None)
    oe, o1, o2 = orc.dist_backward(kind, gout, e, q1, q2)
    assert_close(ge.cpu().numpy(), oe, 4 * rel, "gent")
    assert_close(g1.cpu().numpy(), o1, 4 * rel, "gq1")
    if t2 is not None:
        assert_close(g2.cpu().numpy(), o2, 4 * rel, "gq2")


def test_tie_conventions_on_device():
    from smore_amd import extlib_hip as ext
    cases = [  # kind, e, c, o, expected (ge, gc, go) for gout = 2
        ("l1", 0.5, 0.5, None, (-2.0, 2.0, None)),
        ("box_out", 1.0, 0.75, 0.25, (2.0, -2.0, -2.0)),
        ("box_out", 1.0, 0.75, 0.5, (0.0, 0.0, 0.0)),
        ("box_out", 1.0, 1.0, 0.0, (-2.0, 2.0, -2.0)),
        ("box_in", 1.0, 0.75, 0.25, (0.0, 0.0, 2.0)),
        ("box_in", 0.5, 0.75, 0.5, (-2.0, 2.0, 0.0)),
        ("box_in", 1.0, 0.75, -0.5, (0.0, 0.0, -2.0)),
        ("box_in", 1.0, 1.0, 0.5, (2.0, -2.0, 0.0)),
    ]
    for dtype in (torch.float32, torch.float64):
        for kind, e, c, o, want in cases:
            one = lambda v: None if v is None else torch.tensor([[[v]]], dtype=dtype, device="cuda")
            te, tc, to = one(e), one(c), one(o)
            g = torch.tensor([[2.0]], dtype=dtype, device="cuda")
            ge, gc = torch.empty_like(te), torch.empty_like(tc)
            go = None if to is None else torch.empty_like(to)
            ext.dist_backward(kind, g, te, tc, to, ge, gc, go, to is not None)
            got = (ge.item(), gc.item(), None if go is None else go.item())
            assert got == want, (kind, e, c, o, got, want)


@pytest.mark.parametrize("name", ["l1", "l2", "box", "rotate", "beta_kl", "complex", "distmult"])
def test_reference_smoke_shapes_through_autograd(name):
    """entity [30,1,400] x query [1,20,400 or 200], loss = sum(d^2) * 3.14, seed 1 -- the
    shapes of the reference's own test_* functions (e.g. dist_func/box_dist.py:100-123),
    fast operator against its pure-torch twin and against the oracle."""
    from smore_amd.torchext import ext_ops
    from smore_amd.torchext.dist_func import beta_dist, box_dist, complex_dist, distmult_dist, l1_dist, l2_dist, rotate_dist
    torch.manual_seed(1)
    two = name in ("rotate", "beta_kl", "complex")
    qd = 200 if two else 400
    ent = torch.randn(30, 1, 400)
    qa, qb = torch.randn(1, 20, qd), torch.randn(1, 20, qd)
    if name == "beta_kl":
        ent, qa, qb = (torch.clamp(t + 1, 0.05, 1e9) for t in (ent, qa, qb))
    params = [torch.nn.Parameter(t.cuda()) for t in ((ent, qa) if name in ("l1", "l2", "distmult") else (ent, qa, qb))]
    fast, slow = {
        "l1": (ext_ops.l1_dist, l1_dist.naive_l1),
        "l2": (ext_ops.l2_dist, l2_dist.naive_l2),
        "box": (lambda e, c, o: 24 - ext_ops.box_dist_out(e, c, o) - ext_ops.box_dist_in(e, c, o),
                lambda e, c, o: 24 - box_dist.naive_box_dist_out(e, c, o) - box_dist.naive_box_dist_in(e, c, o)),
        "rotate": (ext_ops.rotate_dist, rotate_dist.naive_rotate_dist),
        "beta_kl": (lambda e, a, b: ext_ops.beta_kl(e, ext_ops.BetaDist(a, b)),
                    lambda e, a, b: beta_dist.naive_beta_kl(e, ext_ops.BetaDist(a, b))),
        "complex": (ext_ops.complex_sim, complex_dist.naive_complex_sim),
        "distmult": (ext_ops.distmult_sim, distmult_dist.naive_innerprod),
    }[name]
    results = []
    for fn in (fast, slow):
        for p in params:
            p.grad = None
        d = fn(*params)
        assert d.shape == (30, 20)
        loss = torch.sum(d ** 2) * 3.14
        loss.backward()
        results.append((loss.item(), [p.grad.detach().cpu().numpy().copy() for p in params]))
    (l_fast, g_fast), (l_slow, g_slow) = results
    assert abs(l_fast - l_slow) <= 1e-5 * abs(l_slow)
    for a, b in zip(g_fast, g_slow):
        assert_close(a, b, 2e-5, f"{name} grad vs torch twin")


def test_four_dim_query_is_looped_over_branches():
    from smore_amd.torchext import ext_ops
    rng = np.random.default_rng(3)
    ent = torch.tensor(rng.standard_normal((5, 7, 16)), dtype=torch.float32, device="cuda", requires_grad=True)
    c = torch.tensor(rng.standard_normal((5, 3, 1, 16)), dtype=torch.float32, device="cuda", requires_grad=True)
    o = torch.tensor(np.abs(rng.standard_normal((5, 3, 1, 16))), dtype=torch.float32, device="cuda", requires_grad=True)
    d = ext_ops.box_dist_out(ent, c, o)
    assert d.shape == (5, 3, 7)
    want = torch.relu((ent.unsqueeze(1) - c).abs() - o).sum(-1)
    assert torch.allclose(d, want, rtol=1e-5, atol=1e-5)
    d.sum().backward()
    ge = ent.grad.clone()
    ent.grad = None
    want.sum().backward()
    assert torch.allclose(ge, ent.grad, rtol=1e-5, atol=1e-5)


def test_precondition_errors():
    from smore_amd import _lib, extlib_hip as ext
    from smore_amd.torchext import ext_ops
    e = torch.zeros(4, 3, 8, device="cuda")
    with pytest.raises(AssertionError):
        ext_ops.l1_dist(e, torch.zeros(4, 1, 7, device="cuda"))      # last dim mismatch
    with pytest.raises(AssertionError):
        ext_ops.l1_dist(e, torch.zeros(3, 1, 8, device="cuda"))      # 4 vs 3 do not divide
    with pytest.raises(AssertionError):
        ext_ops.l1_dist(e.transpose(0, 1), torch.zeros(3, 1, 8, device="cuda"))  # not contiguous
    with pytest.raises(_lib.SmxError):
        ext.dist_forward("nonsense", e, e, None, torch.zeros(4, 3, device="cuda"), False)
    with pytest.raises(_lib.SmxError):
        ext.l1_dist_forward(torch.zeros(4, 3, 8), torch.zeros(4, 1, 8), torch.zeros(4, 3))  # CPU tensors
