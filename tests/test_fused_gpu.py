"""Gather-fused path (score forward, query backward, segment plan, entity backward + sparse Adam)
through the C ABI against the CPU oracle.  Integer results are compared bit for bit, floating
point ones to the 1e-5 bar of tests/util.py."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests.util import REL_F32, assert_close, record_headroom, seed

pytestmark = pytest.mark.gpu

GAMMA = {"l1": 12.0, "l2": 12.0, "box": 24.0, "rotate": 9.0, "beta_kl": 60.0, "complex": 0.0, "distmult": 0.0,
         "complex_norm": 0.0,   # complex with unit-length row halves (complex.py:142-146)
         "distmult_norm": 0.0}  # distmult with unit-length rows (distmult.py:129-130)


def make_problem(model, n, b, k, dim, rng, zipf=None, scale=0.07):
    """Table, queries, ids and upstream gradient of one step, as fp32-representable float64."""
    mul = 2 if model in ("rotate", "beta_kl", "complex") else 1
    f32 = lambda x: x.astype(np.float32).astype(np.float64)
    if model == "beta_kl":
        def beta(*s):
            x = rng.standard_normal(s)
            return np.clip(1 + np.where(x > 0, x, np.expm1(x)), 0.05, 1e9)
        table, q1, q2 = beta(n, dim * mul), beta(b, dim), beta(b, dim)
    else:
        table = rng.uniform(-scale, scale, (n, dim * mul))
        q1 = rng.uniform(-scale, scale, (b, dim))
        q2 = None if model in ("l1", "l2", "distmult") else rng.uniform(-scale, scale, (b, dim))
        if model == "box":
            q2 = np.abs(q2)
    if zipf is None:
        idx = rng.integers(0, n, (b, k))
    else:
        w = 1.0 / np.arange(1, n + 1) ** zipf
        idx = rng.choice(n, size=(b, k), p=w / w.sum())
    gs = rng.standard_normal((b, k))
    return f32(table), f32(q1), None if q2 is None else f32(q2), idx.astype(np.int64), f32(gs)


def _serial_backward(on):
    """smx_set_option(SMX_OPTION_SERIAL_BACKWARD): every kernel of the backward on the caller's stream."""
    from smore_amd import _lib
    _lib.call("smx_set_option", _lib.OPTION_SERIAL_BACKWARD, int(on))


def dev(a, dtype=torch.float32):
    return None if a is None else torch.tensor(a, dtype=dtype, device="cuda")


def run_case(model, n, b, k, dim, zipf=None, cen=0.02, adam_steps=2, lr=1e-3):
    from smore_amd import fused
    rng = np.random.default_rng(seed(model, n, b, k, dim, zipf))
    gamma = GAMMA[model]
    norm = model.endswith("_norm")
    model = model[:-5] if norm else model
    table, q1, q2, idx, gs = make_problem(model, n, b, k, dim, rng, zipf)
    params = fused.score_params(gamma, cen, norm=norm)
    t_table, t_q1, t_q2, t_gs = dev(table), dev(q1), dev(q2), dev(gs)
    t_idx = torch.tensor(idx, device="cuda")
    err = fused.new_error_flag("cuda")

    # forward
    score = fused.score_forward(model, t_table, t_idx, t_q1, t_q2, params, err)
    rows = orc.gather(table, idx).reshape(b, k, -1)
    o_q1 = q1[:, None, :]
    o_q2 = None if q2 is None else q2[:, None, :]
    want = orc.score_forward(model, rows, o_q1, o_q2, gamma, cen, norm=norm)
    # no RMS floor for the scores of the models whose distance is a sum of non-negative terms: every element to 1e-5
    # (a KL divergence or an inner product is a sum of signed terms)
    assert_close(score.cpu().numpy(), want, REL_F32, f"{model} score", rms_floor=model in ("beta_kl", "complex", "distmult"))
    assert err.item() == 0

    # dense layout (idx = None) gives the same scores bit for bit
    t_rows = dev(rows.reshape(b * k, -1))
    score_dense = fused.score_forward(model, t_rows, None, t_q1, t_q2, params)
    assert torch.equal(score_dense, score)

    # query backward
    gq1, gq2 = fused.score_backward_query(model, t_table, t_idx, t_q1, t_q2, score, t_gs, params)
    o_rows, o_g1, o_g2 = orc.score_backward(model, gs, rows, o_q1, o_q2, cen, norm=norm)
    # a query gradient is a sum over K signed terms of size <= |g_k| (unit-bounded derivatives of l1, l2, box,
    # rotate): when it cancels, one fp32 ulp of sum |g_k| is the floor of any summation order
    q_abs = None if model == "beta_kl" else np.abs(gs).sum(axis=1)[:, None] * np.ones((1, dim))
    assert_close(gq1.cpu().numpy(), o_g1[:, 0, :], REL_F32, f"{model} gq1", sum_abs=q_abs)
    if q2 is not None:
        assert_close(gq2.cpu().numpy(), o_g2[:, 0, :], REL_F32, f"{model} gq2", sum_abs=q_abs)

    # plan: integers are bit-exact
    plan = fused.build_plan(t_idx, n, want_inverse=True, err_flag=err)
    uniq, inverse, order, seg_start = orc.merge_indices(idx)
    assert plan.n_uniq == uniq.size
    assert np.array_equal(plan.uniq.cpu().numpy(), uniq)
    assert np.array_equal(plan.inverse.cpu().numpy(), inverse)
    assert np.array_equal(plan.order.cpu().numpy().astype(np.int64), order)
    assert np.array_equal(plan.seg_start[: uniq.size + 1].cpu().numpy().astype(np.int64), seg_start)
    assert np.array_equal(plan.sorted_ids.cpu().numpy().astype(np.int64), idx.reshape(-1)[order])
    assert np.array_equal(plan.seg_of_pos.cpu().numpy().astype(np.int64), inverse[order])
    assert err.item() == 0

    # entity backward: merged gradient only
    merged = torch.full((uniq.size, table.shape[1]), float("nan"), device="cuda")
    fused.score_backward_entity(model, plan, t_table, t_q1, t_q2, score, t_gs, params, merged=merged)
    o_merged = orc.merge_grads(o_rows.reshape(b * k, -1), inverse, uniq.size)
    o_abs = orc.merge_grads(np.abs(o_rows).reshape(b * k, -1), inverse, uniq.size)
    assert_close(merged.cpu().numpy(), o_merged, REL_F32, f"{model} merged entity grad", sum_abs=o_abs)
    assert torch.equal(t_table, dev(table)), "table must not change without Adam"

    # one-call backward (one-pair segments finished by the query-gradient kernel): same values up to the
    # rounding of a contracted multiply-add (the two kernels are compiled separately)
    merged3 = torch.full_like(merged, float("nan"))
    f1, f2 = fused.score_backward_fused(model, plan, t_table, t_idx, t_q1, t_q2, score, t_gs, params, merged=merged3)
    assert_close(f1.cpu().numpy(), gq1.cpu().numpy(), 1e-6, f"{model} gq1, one-call backward", sum_abs=q_abs)
    if gq2 is not None:
        assert_close(f2.cpu().numpy(), gq2.cpu().numpy(), 1e-6, f"{model} gq2, one-call backward", sum_abs=q_abs)
    assert_close(merged3.cpu().numpy(), merged.cpu().numpy(), 1e-6, f"{model} merged, one-call backward")
    assert (plan.pair_seg < 0).sum().item() == int((np.diff(seg_start) == 1).sum())

    # same sum from materialised gradient rows
    merged2 = torch.full_like(merged, float("nan"))
    fused.rows_backward(plan, dev(o_rows.reshape(b * k, -1)), merged=merged2)
    assert_close(merged2.cpu().numpy(), o_merged, REL_F32, f"{model} merged (rows source)", sum_abs=o_abs)

    # fused Adam, several steps so m and v are non-trivial.  Adam divides by sqrt(v): where a summed
    # gradient cancels to ~eps its update is ill-conditioned, so (a) the Adam arithmetic is checked step
    # by step from the device's own state and merged gradient, to the 1e-5 bar, and (b) the end-to-end
    # trajectory against the float64 oracle is checked to 1e-5 on all but a sliver of such elements (at most 2 in
    # 10,000), which must still be within a tenth of a learning-rate step per step taken.
    w_o, m_o, v_o = table.copy(), np.zeros_like(table), np.zeros_like(table)
    t_m, t_v = torch.zeros_like(t_table), torch.zeros_like(t_table)
    touched = np.zeros(n, bool)
    touched[uniq] = True
    for step in range(1, adam_steps + 1):
        sc = fused.score_forward(model, t_table, t_idx, t_q1, t_q2, params)
        fused.score_backward_entity(model, plan, t_table, t_q1, t_q2, sc, t_gs, params, merged=merged)
        w_s, m_s, v_s = (x.cpu().numpy().astype(np.float64) for x in (t_table, t_m, t_v))
        orc.adam_rows(w_s, m_s, v_s, uniq, merged.cpu().numpy().astype(np.float64), lr, step)
        c_table, c_m, c_v = t_table.clone(), t_m.clone(), t_v.clone()
        fused.score_backward_entity(model, plan, t_table, t_q1, t_q2, sc, t_gs, params, m=t_m, v=t_v,
                                    adam=fused.adam_params(lr, step))
        fused.score_backward_fused(model, plan, c_table, t_idx, t_q1, t_q2, sc, t_gs, params, m=c_m, v=c_v,
                                   adam=fused.adam_params(lr, step))
        for got, ref, what in ((c_table, t_table, "w"), (c_m, t_m, "m"), (c_v, t_v, "v")):
            assert_close(got.cpu().numpy()[touched], ref.cpu().numpy()[touched], 2e-6, f"{model} one-call backward: {what}")
            assert torch.equal(got[torch.tensor(~touched, device="cuda")], ref[torch.tensor(~touched, device="cuda")])
        assert_close(t_table.cpu().numpy()[touched], w_s[touched], REL_F32, f"{model} Adam step {step}: w")
        assert_close(t_m.cpu().numpy()[touched], m_s[touched], REL_F32, f"{model} Adam step {step}: m")
        assert_close(t_v.cpu().numpy()[touched], v_s[touched], REL_F32, f"{model} Adam step {step}: v", rms_floor=False)
        orc.train_step(model, w_o, m_o, v_o, idx, o_q1, o_q2, gs, gamma, cen, lr, step, norm=norm)
    got_w = t_table.cpu().numpy()
    err = np.abs(got_w - w_o)[touched]
    tol = REL_F32 * np.maximum(np.abs(w_o[touched]), np.sqrt(np.mean(w_o[touched] ** 2)))
    # (worst seen over every case of this file: a share of 1.6e-5 and 0.003 lr per step)
    assert (err > tol).mean() < 2e-4 and err.max() < 0.1 * lr * adam_steps, (err.max(), (err > tol).mean())
    record_headroom(f"{model} w trajectory: share of elements outside 1e-5 / 2e-4, worst error / (0.1 lr steps)",
                    (err > tol).mean() / 2e-4, err.max() / (0.1 * lr * adam_steps))
    assert_close(t_m.cpu().numpy()[touched], m_o[touched], 5 * REL_F32, f"{model} m trajectory")
    assert np.array_equal(got_w[~touched], table[~touched].astype(np.float32)), "untouched rows must stay bit-identical"
    assert not t_m.cpu().numpy()[~touched].any() and not t_v.cpu().numpy()[~touched].any()


@pytest.mark.parametrize("model", list(GAMMA))
@pytest.mark.parametrize("shape", [
    (500, 6, 10, 32),      # small, float4 path
    (300, 5, 7, 13),       # odd dim: scalar path
    (2000, 16, 128, 200),  # config-1-like row length
    (40, 8, 64, 16),       # 40 ids over 512 pairs: every segment is long
    (5000, 3, 300, 400),   # two column iterations per lane
])
def test_fused_step_matches_oracle(model, shape):
    n, b, k, dim = shape
    run_case(model, n, b, k, dim)


def _sweep_cases(count=20):
    """Seeded random shapes: few ids (long segments) to many, K below / across / above the 64-pair batch,
    dims on and off the float4 path and across the 256- and 512-float column groups."""
    rng = np.random.default_rng(20240)
    models = list(GAMMA)
    cases = []
    for i in range(count):
        dim = int(rng.choice([4, 12, 31, 64, 100, 200, 260, 400, 516]))
        if dim % 4 and dim > 256:
            dim -= dim % 4
        b, k = int(rng.integers(1, 12)), int(rng.choice([1, 3, 63, 64, 65, 130, 257]))
        n = int(rng.choice([7, 50, 600, 20000]))
        cases.append((models[i % len(models)], n, b, k, dim, None if i % 3 else 1.1))
    return cases


@pytest.mark.parametrize("case", _sweep_cases(), ids=lambda c: "-".join(str(x) for x in c))
def test_fused_step_random_shapes(case):
    model, n, b, k, dim, zipf = case
    run_case(model, n, b, k, dim, zipf=zipf, adam_steps=1)


def test_rotate_zero_modulus_features_follow_the_eps_convention():
    """Features where entity and query coincide: the modulus is sqrt(0 + 1e-20) and its derivative
    0 * rsqrt(1e-20) = 0 (cuda_math_ext.h:100-118) -- finite, no NaN, on the fused and the dense path."""
    from smore_amd import fused
    from smore_amd import extlib_hip as ext
    rng = np.random.default_rng(2)
    n, b, k, dim = 30, 3, 9, 24
    table, q1, q2, idx, gs = make_problem("rotate", n, b, k, dim, rng)
    table[5, :dim] = q1[0]; table[5, dim:] = q2[0]          # entity 5 equals query 0 in every feature
    table[6, :7] = q1[1, :7]; table[6, dim:dim + 7] = q2[1, :7]   # entity 6 equals query 1 in seven of them
    idx[0, :2] = 5
    idx[1, 3] = 6
    params = fused.score_params(GAMMA["rotate"], 0.0)
    t_table, t_q1, t_q2, t_gs, t_idx = dev(table), dev(q1), dev(q2), dev(gs), torch.tensor(idx, device="cuda")
    score = fused.score_forward("rotate", t_table, t_idx, t_q1, t_q2, params)
    rows = orc.gather(table, idx).reshape(b, k, -1)
    want = orc.score_forward("rotate", rows, q1[:, None], q2[:, None], GAMMA["rotate"], 0.0)
    assert_close(score.cpu().numpy(), want, REL_F32, "rotate score with zero-modulus features")
    assert abs(GAMMA["rotate"] - score[0, 0].item() - dim * 1e-10) < 1e-12 + 1e-6 * dim * 1e-10 + 1e-6  # gamma - dim * sqrt(eps)
    gq1, gq2 = fused.score_backward_query("rotate", t_table, t_idx, t_q1, t_q2, score, t_gs, params)
    o_rows, o_g1, o_g2 = orc.score_backward("rotate", gs, rows, q1[:, None], q2[:, None], 0.0)
    assert torch.isfinite(gq1).all() and torch.isfinite(gq2).all()
    assert_close(gq1.cpu().numpy(), o_g1[:, 0], REL_F32, "gq1")
    assert_close(gq2.cpu().numpy(), o_g2[:, 0], REL_F32, "gq2")
    plan = fused.build_plan(t_idx, n)
    merged = torch.empty((plan.n_uniq, 2 * dim), device="cuda")
    fused.score_backward_entity("rotate", plan, t_table, t_q1, t_q2, score, t_gs, params, merged=merged)
    assert torch.isfinite(merged).all()
    uniq, inverse, _, _ = orc.merge_indices(idx)
    o_merged = orc.merge_grads(o_rows.reshape(b * k, -1), inverse, uniq.size)
    o_abs = orc.merge_grads(np.abs(o_rows).reshape(b * k, -1), inverse, uniq.size)
    assert_close(merged.cpu().numpy(), o_merged, REL_F32, "merged", sum_abs=o_abs)
    # the dense operator on the same rows
    t_rows = dev(rows)
    dst = torch.empty((b, k), device="cuda")
    ext.dist_forward("rotate", t_rows, t_q1[:, None].contiguous(), t_q2[:, None].contiguous(), dst, True)
    assert_close(dst.cpu().numpy(), GAMMA["rotate"] - want, REL_F32, "dense rotate distance")


@pytest.mark.parametrize("model", ["box", "rotate"])
def test_segments_crossing_many_tiles(model):
    """Zipf ids with a head id that owns ~20% of 16k pairs: segments span many tiles of the
    entity pass, the partial-row path and its fixed-order combine are exercised."""
    run_case(model, 3000, 32, 512, 64, zipf=1.3)


def test_large_pair_count_uses_long_tiles():
    """2.2M pairs: the entity pass switches to tiles longer than one wavefront batch."""
    run_case("box", 100000, 1024, 2176, 8, zipf=1.1, adam_steps=1)


def test_dim_1000_rotate_row():
    run_case("rotate", 3000, 4, 33, 500, adam_steps=1)


def test_regularizer_prologue_beta():
    """BetaE stores raw values; clamp(x + 1, 0.05, 1e9) is applied after the gather and its
    backward masks the gradient where the clamp is active."""
    from smore_amd import fused
    rng = np.random.default_rng(77)
    n, b, k, dim = 400, 6, 20, 24
    raw = (rng.standard_normal((n, 2 * dim)) * 1.5).astype(np.float32).astype(np.float64)
    f = lambda *s: np.clip(1 + rng.standard_normal(s), 0.05, 1e9).astype(np.float32).astype(np.float64)
    qa, qb = f(b, dim), f(b, dim)
    idx = rng.integers(0, n, (b, k))
    gs = rng.standard_normal((b, k)).astype(np.float32).astype(np.float64)
    params = fused.score_params(60.0, 0.0, regularizer=(1.0, 0.05, 1e9))
    t_raw, t_qa, t_qb, t_gs = dev(raw), dev(qa), dev(qb), dev(gs)
    t_idx = torch.tensor(idx, device="cuda")
    score = fused.score_forward("beta_kl", t_raw, t_idx, t_qa, t_qb, params)
    reg = orc.regularizer(raw)
    assert (raw + 1 < 0.05).any(), "the case must hit the clamp"
    rows = orc.gather(reg, idx).reshape(b, k, -1)
    want = orc.score_forward("beta_kl", rows, qa[:, None], qb[:, None], 60.0)
    assert_close(score.cpu().numpy(), want, REL_F32, "regularised beta score")
    g_rows, g_a, g_b = orc.score_backward("beta_kl", gs, rows, qa[:, None], qb[:, None])
    gq1, gq2 = fused.score_backward_query("beta_kl", t_raw, t_idx, t_qa, t_qb, score, t_gs, params)
    assert_close(gq1.cpu().numpy(), g_a[:, 0], REL_F32, "gq alpha")
    assert_close(gq2.cpu().numpy(), g_b[:, 0], REL_F32, "gq beta")
    plan = fused.build_plan(t_idx, n, want_inverse=True)
    uniq, inverse, _, _ = orc.merge_indices(idx)
    merged = torch.empty((uniq.size, 2 * dim), device="cuda")
    fused.score_backward_entity("beta_kl", plan, t_raw, t_qa, t_qb, score, t_gs, params, merged=merged)
    o_merged = orc.merge_grads(g_rows.reshape(b * k, -1), inverse, uniq.size)
    mask = ((raw[uniq] + 1 >= 0.05) & (raw[uniq] + 1 <= 1e9))
    assert_close(merged.cpu().numpy(), o_merged * mask, REL_F32, "masked entity gradient")


def test_out_of_range_id_sets_the_flag():
    from smore_amd import fused
    t = torch.zeros(10, 8, device="cuda")
    q = torch.zeros(2, 8, device="cuda")
    err = fused.new_error_flag("cuda")
    idx = torch.tensor([[0, 3], [10, 1]], device="cuda")
    fused.score_forward("l1", t, idx, q, None, fused.score_params(1.0), err)
    assert err.item() == 1
    err.zero_()
    fused.build_plan(torch.tensor([[0, -1]], device="cuda"), 10, err_flag=err)
    assert err.item() == 1


@pytest.mark.parametrize("n_pairs_shape", [(6, 40), (40, 1024)])
def test_out_of_range_ids_update_no_row(n_pairs_shape):
    """Pairs whose id lies outside the table are kept out of the plan's segments: n_uniq / uniq are those of the
    valid ids, no row -- row 0 least of all -- is updated for them, and the rows of the valid ids get what the
    oracle gives when the bad pairs contribute nothing."""
    from smore_amd import fused
    b, k = n_pairs_shape
    n, dim, lr = 3000, 64, 1e-3
    rng = np.random.default_rng(seed("bad ids", b, k))
    table, q1, q2, idx, gs = make_problem("box", n, b, k, dim, rng, zipf=1.05)
    idx = np.maximum(idx, 1)                                   # row 0 is named by no valid pair
    bad = rng.random((b, k)) < 0.03
    bad[0, 0] = bad[-1, -1] = True
    idx_bad = idx.copy()
    idx_bad[bad] = rng.choice([-1, n, n + 7, 1 << 40, -(1 << 35)], size=int(bad.sum()))
    t_q1, t_q2, t_gs = dev(q1), dev(q2), dev(gs)
    t_idx = torch.tensor(idx_bad, device="cuda")
    params = fused.score_params(24.0, 0.02)
    err = fused.new_error_flag("cuda")
    plan = fused.build_plan(t_idx, n, want_inverse=True, err_flag=err)
    assert err.item() == 1
    uniq = np.unique(idx[~bad])
    assert plan.n_uniq == uniq.size and np.array_equal(plan.uniq.cpu().numpy(), uniq)
    inv = plan.inverse.cpu().numpy().reshape(b, k)
    assert np.array_equal(inv[~bad], np.searchsorted(uniq, idx[~bad])) and (inv[bad] == uniq.size).all()
    assert not (plan.pair_seg.cpu().numpy().reshape(b, k)[bad] < 0).any()
    # the oracle's step on the valid pairs: bad pairs moved onto a valid id of their query with zero upstream gradient
    idx_ref, gs_ref = idx_bad.copy(), gs.copy()
    idx_ref[bad] = np.broadcast_to(uniq[:1], (b, k))[bad]
    gs_ref[bad] = 0.0
    w_o, m_o, v_o = table.copy(), np.zeros_like(table), np.zeros_like(table)
    orc.train_step("box", w_o, m_o, v_o, idx_ref, q1[:, None], q2[:, None], gs_ref, 24.0, 0.02, lr, 1)
    touched = np.zeros(n, bool)
    touched[uniq] = True
    for one_call in (False, True):
        t_table = dev(table)
        t_m, t_v = torch.zeros_like(t_table), torch.zeros_like(t_table)
        codes = fused.new_codes("box", t_table, t_idx, t_q1)
        score = fused.score_forward("box", t_table, t_idx, t_q1, t_q2, params, err, codes=codes)
        if one_call:
            fused.score_backward_fused("box", plan, t_table, t_idx, t_q1, t_q2, score, t_gs, params, m=t_m, v=t_v,
                                       adam=fused.adam_params(lr, 1), codes=codes)
        else:
            fused.score_backward_entity("box", plan, t_table, t_q1, t_q2, score, t_gs, params, m=t_m, v=t_v,
                                        adam=fused.adam_params(lr, 1))
        w, m, v = (x.cpu().numpy() for x in (t_table, t_m, t_v))
        assert np.array_equal(w[~touched], table[~touched].astype(np.float32)), "a row without a valid pair changed"
        assert not m[~touched].any() and not v[~touched].any()
        # (the row that collected the moved pairs in the oracle got zero gradient from them: nothing was added)
        assert_close(m[touched], m_o[touched], 5 * REL_F32, "first moment of the valid rows")
        assert_close(v[touched], v_o[touched], 5 * REL_F32, "second moment of the valid rows")


def test_entity_pass_is_deterministic():
    from smore_amd import fused
    rng = np.random.default_rng(5)
    table, q1, q2, idx, gs = make_problem("box", 200, 16, 256, 64, rng, zipf=1.2)
    t_table, t_q1, t_q2, t_gs = dev(table), dev(q1), dev(q2), dev(gs)
    t_idx = torch.tensor(idx, device="cuda")
    params = fused.score_params(24.0, 0.02)
    score = fused.score_forward("box", t_table, t_idx, t_q1, t_q2, params)
    outs = []
    for _ in range(3):
        plan = fused.build_plan(t_idx, 200)
        merged = torch.empty((plan.n_uniq, 64), device="cuda")
        fused.score_backward_entity("box", plan, t_table, t_q1, t_q2, score, t_gs, params, merged=merged)
        outs.append(merged.clone())
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])


def test_argument_errors():
    from smore_amd import _lib, fused
    t = torch.zeros(10, 8, device="cuda")
    q = torch.zeros(2, 8, device="cuda")
    idx = torch.zeros(2, 3, dtype=torch.int64, device="cuda")
    with pytest.raises(_lib.SmxError):
        fused.score_forward("nope", t, idx, q, None, fused.score_params(1.0))
    with pytest.raises(_lib.SmxError):
        fused.score_forward("box", t, idx, q, None, fused.score_params(1.0))       # box needs two queries
    with pytest.raises(_lib.SmxError):
        fused.score_forward("l1", t, idx, torch.zeros(2, 7, device="cuda"), None, fused.score_params(1.0))
    with pytest.raises(_lib.SmxError):
        fused.score_forward("l1", t, idx.int(), q, None, fused.score_params(1.0))  # ids must be int64
    with pytest.raises(_lib.SmxError):
        fused.score_forward("l1", torch.zeros(10, 4100, device="cuda"), idx, torch.zeros(2, 4100, device="cuda"),
                            None, fused.score_params(1.0))                          # row too long for the fused path
    plan = fused.build_plan(idx, 10)
    with pytest.raises(_lib.SmxError):
        fused.score_backward_entity("l1", plan, t, q, None, torch.zeros(2, 3, device="cuda"),
                                    torch.zeros(2, 3, device="cuda"), fused.score_params(1.0))  # nothing requested


def test_box_tie_conventions_through_the_fused_path():
    """The fused box kernels use a rearranged derivative; at ties it must still give the values of
    the reference functors (dist_kernel.h:68-104): sign(0) = -1 outside, gradient passes at
    |e-c| == o, e == c inside the box, negative offsets."""
    from smore_amd import fused
    cases = [  # e, c, o
        (1.0, 0.75, 0.25), (1.0, 0.75, 0.5), (1.0, 1.0, 0.0), (0.5, 0.75, 0.5), (1.0, 0.75, -0.5),
        (1.0, 1.0, 0.5), (0.25, 0.75, 0.25), (1.0, 1.0, -0.5), (0.75, 1.0, 0.0),
    ]
    n = len(cases)
    table = np.array([[e] * 4 for e, _, _ in cases], dtype=np.float64)      # one entity row per case
    q1 = np.array([[c] * 4 for _, c, _ in cases], dtype=np.float64)          # one query per case
    q2 = np.array([[o] * 4 for _, _, o in cases], dtype=np.float64)
    idx = np.arange(n, dtype=np.int64)[:, None]                              # pair (i, i)
    gs = np.full((n, 1), 2.0)
    params = fused.score_params(24.0, 0.5)
    t_table, t_q1, t_q2, t_gs = dev(table), dev(q1), dev(q2), dev(gs)
    t_idx = torch.tensor(idx, device="cuda")
    score = fused.score_forward("box", t_table, t_idx, t_q1, t_q2, params)
    rows = table[:, None, :]
    want = orc.score_forward("box", rows, q1[:, None], q2[:, None], 24.0, 0.5)
    assert np.array_equal(score.cpu().numpy().astype(np.float64), want)
    g_rows, g_c, g_o = orc.score_backward("box", gs, rows, q1[:, None], q2[:, None], 0.5)
    gq1, gq2 = fused.score_backward_query("box", t_table, t_idx, t_q1, t_q2, score, t_gs, params)
    assert np.array_equal(gq1.cpu().numpy().astype(np.float64), g_c[:, 0])
    assert np.array_equal(gq2.cpu().numpy().astype(np.float64), g_o[:, 0])
    plan = fused.build_plan(t_idx, n)
    merged = torch.empty((n, 4), device="cuda")
    fused.score_backward_entity("box", plan, t_table, t_q1, t_q2, score, t_gs, params, merged=merged)
    assert np.array_equal(merged.cpu().numpy().astype(np.float64), g_rows[:, 0])


def test_one_call_backward_with_many_queries_takes_the_one_pair_shortcut():
    """With query tensors above 4 MiB the one-call backward finishes one-pair segments in the
    query-gradient kernel; results must still equal the two separate calls."""
    from smore_amd import fused
    rng = np.random.default_rng(12)
    n, b, k, dim = 60000, 4200, 6, 128   # 4200 x 2 x 128 floats = 4.3 MB of queries
    table, q1, q2, idx, gs = make_problem("box", n, b, k, dim, rng)
    t_table, t_q1, t_q2, t_gs = dev(table), dev(q1), dev(q2), dev(gs)
    t_idx = torch.tensor(idx, device="cuda")
    params = fused.score_params(24.0, 0.02)
    plan = fused.build_plan(t_idx, n)
    assert 0.3 < (plan.pair_seg < 0).float().mean().item() < 0.9
    score = fused.score_forward("box", t_table, t_idx, t_q1, t_q2, params)
    gq1, gq2 = fused.score_backward_query("box", t_table, t_idx, t_q1, t_q2, score, t_gs, params)
    w_a, m_a, v_a = t_table.clone(), torch.zeros_like(t_table), torch.zeros_like(t_table)
    w_b, m_b, v_b = t_table.clone(), torch.zeros_like(t_table), torch.zeros_like(t_table)
    fused.score_backward_entity("box", plan, w_a, t_q1, t_q2, score, t_gs, params, m=m_a, v=v_a,
                                adam=fused.adam_params(1e-3, 1))
    f1, f2 = fused.score_backward_fused("box", plan, w_b, t_idx, t_q1, t_q2, score, t_gs, params, m=m_b, v=v_b,
                                        adam=fused.adam_params(1e-3, 1))
    assert_close(f1.cpu().numpy(), gq1.cpu().numpy(), 1e-6, "gq1")
    assert_close(f2.cpu().numpy(), gq2.cpu().numpy(), 1e-6, "gq2")
    assert_close(m_b.cpu().numpy(), m_a.cpu().numpy(), 2e-6, "m")
    assert_close(v_b.cpu().numpy(), v_a.cpu().numpy(), 2e-6, "v")
    assert_close(w_b.cpu().numpy(), w_a.cpu().numpy(), 2e-6, "w")
    merged_a = torch.empty((plan.n_uniq, dim), device="cuda")
    merged_b = torch.full_like(merged_a, float("nan"))
    fused.score_backward_entity("box", plan, t_table, t_q1, t_q2, score, t_gs, params, merged=merged_a)
    fused.score_backward_fused("box", plan, t_table, t_idx, t_q1, t_q2, score, t_gs, params, merged=merged_b)
    assert_close(merged_b.cpu().numpy(), merged_a.cpu().numpy(), 1e-6, "merged")


@pytest.mark.parametrize("dim", [128, 400, 30])
def test_sign_codes_give_the_bits_of_the_query_row_path(dim):
    """With many queries the box backward leaves per-pair sign codes for the entity pass
    (smx_fused_workspace_bytes); without the extra workspace the entity pass re-reads the query rows.
    Both sum the same +-c terms in the same order: the merged rows must be equal bit for bit, long
    segments, repeated (entity, query) pairs and all."""
    from smore_amd import fused
    rng = np.random.default_rng(dim)
    b = (4 << 20) // (2 * 4 * dim) + 64
    n, k = 3000, 6
    table, q1, q2, idx, gs = make_problem("box", n, b, k, dim, rng, zipf=1.2)
    idx[::3, 1] = idx[::3, 0]            # the same entity twice under one query
    t_table, t_q1, t_q2, t_gs = dev(table), dev(q1), dev(q2), dev(gs)
    t_idx = torch.tensor(idx, device="cuda")
    params = fused.score_params(24.0, 0.02)
    plan = fused.build_plan(t_idx, n)
    score = fused.score_forward("box", t_table, t_idx, t_q1, t_q2, params)
    saved = fused.new_codes("box", t_table, t_idx, t_q1)
    assert saved is not None and saved.numel() == b * k * 64 * (2 if dim == 400 else 1)
    score_saving = fused.score_forward("box", t_table, t_idx, t_q1, t_q2, params, codes=saved)
    assert torch.equal(score_saving, score)
    out = {}
    for codes in (False, True, "forward"):
        merged = torch.full((plan.n_uniq, dim), float("nan"), device="cuda")
        g1, g2 = fused.score_backward_fused("box", plan, t_table, t_idx, t_q1, t_q2, score, t_gs, params,
                                            merged=merged, sign_codes=codes is True,
                                            codes=saved if codes == "forward" else None)
        out[codes] = (merged.cpu().numpy(), g1.cpu().numpy(), g2.cpu().numpy())
    for how in (True, "forward"):
        assert np.array_equal(out[how][0], out[False][0]), how
        assert_close(out[how][1], out[False][1], 1e-6, "gq1")
        assert_close(out[how][2], out[False][2], 1e-6, "gq2")
    # Adam from the forward's codes against Adam from the recomputed derivative
    state = {}
    for how in (False, "forward"):
        w, m, v = t_table.clone(), torch.zeros_like(t_table), torch.zeros_like(t_table)
        fused.score_backward_fused("box", plan, w, t_idx, t_q1, t_q2, score, t_gs, params, m=m, v=v,
                                   adam=fused.adam_params(1e-3, 1), sign_codes=False,
                                   codes=saved if how == "forward" else None)
        state[how] = (w.cpu().numpy(), m.cpu().numpy(), v.cpu().numpy())
    for a, b_, what in zip(state["forward"], state[False], "wmv"):
        assert_close(a, b_, 2e-6, what)
    g_rows, _, _ = orc.score_backward("box", gs, table[idx], q1[:, None], q2[:, None], 0.02)
    uniq, inv = np.unique(idx.reshape(-1), return_inverse=True)
    want = np.zeros((len(uniq), dim))
    np.add.at(want, inv, g_rows.reshape(-1, dim))
    sum_abs = np.zeros((len(uniq), dim))
    np.add.at(sum_abs, inv, np.abs(g_rows.reshape(-1, dim)))
    assert_close(out[True][0], want, REL_F32, "merged vs oracle", sum_abs=sum_abs)


@pytest.mark.parametrize("b,k,dim", [(3, 37, 200), (5, 100, 64), (2, 1, 8), (1, 300, 6), (9, 17, 512), (4, 65, 31)])
def test_forward_codes_on_odd_shapes(b, k, dim):
    """Codes saved by the forward for batch shapes that do not fill the 16-pair staging groups, the
    64-pair batches or the float4 columns; the backward from codes against the recomputing backward."""
    from smore_amd import fused
    rng = np.random.default_rng(b * 100 + k)
    n = 50
    table, q1, q2, idx, gs = make_problem("box", n, b, k, dim, rng)
    t_table, t_q1, t_q2, t_gs = dev(table), dev(q1), dev(q2), dev(gs)
    t_idx = torch.tensor(idx, device="cuda")
    params = fused.score_params(24.0, 0.02)
    plan = fused.build_plan(t_idx, n)
    saved = fused.new_codes("box", t_table, t_idx, t_q1)
    score = fused.score_forward("box", t_table, t_idx, t_q1, t_q2, params, codes=saved)
    assert torch.equal(score, fused.score_forward("box", t_table, t_idx, t_q1, t_q2, params))
    res = {}
    for how in ("recompute", "codes"):
        merged = torch.full((plan.n_uniq, dim), float("nan"), device="cuda")
        g1, g2 = fused.score_backward_fused("box", plan, t_table, t_idx, t_q1, t_q2, score, t_gs, params,
                                            merged=merged, sign_codes=False, codes=saved if how == "codes" else None)
        res[how] = (merged.cpu().numpy(), g1.cpu().numpy(), g2.cpu().numpy())
    assert np.array_equal(res["codes"][0], res["recompute"][0])
    assert_close(res["codes"][1], res["recompute"][1], 1e-6, "gq1")
    assert_close(res["codes"][2], res["recompute"][2], 1e-6, "gq2")
    # the two separate entry points accept the forward's codes too
    s1, s2 = fused.score_backward_query("box", t_table, t_idx, t_q1, t_q2, score, t_gs, params, codes=saved)
    assert_close(s1.cpu().numpy(), res["recompute"][1], 1e-6, "gq1 (separate call, codes)")
    assert_close(s2.cpu().numpy(), res["recompute"][2], 1e-6, "gq2 (separate call, codes)")
    merged_s = torch.full((plan.n_uniq, dim), float("nan"), device="cuda")
    fused.score_backward_entity("box", plan, t_table, t_q1, t_q2, score, t_gs, params, merged=merged_s, codes=saved)
    assert np.array_equal(merged_s.cpu().numpy(), res["recompute"][0])
    w, m, v = t_table.clone(), torch.zeros_like(t_table), torch.zeros_like(t_table)
    w2, m2, v2 = t_table.clone(), torch.zeros_like(t_table), torch.zeros_like(t_table)
    fused.score_backward_fused("box", plan, w, t_idx, t_q1, t_q2, score, t_gs, params, m=m, v=v,
                               adam=fused.adam_params(1e-3, 1), codes=saved)
    fused.score_backward_fused("box", plan, w2, t_idx, t_q1, t_q2, score, t_gs, params, m=m2, v=v2,
                               adam=fused.adam_params(1e-3, 1), sign_codes=False)
    assert_close(m.cpu().numpy(), m2.cpu().numpy(), 2e-6, "m")
    assert_close(w.cpu().numpy(), w2.cpu().numpy(), 2e-6, "w")


def test_sign_codes_keep_the_tie_conventions():
    """Ties (e == c, |e - c| == o, negative offsets) through the coded path: every pair of the tie table,
    under enough queries for the codes to be used, must give the oracle's rows exactly."""
    from smore_amd import fused
    cases = [  # e, c, o
        (1.0, 0.75, 0.25), (1.0, 0.75, 0.5), (1.0, 1.0, 0.0), (0.5, 0.75, 0.5), (1.0, 0.75, -0.5),
        (1.0, 1.0, 0.5), (0.25, 0.75, 0.25), (1.0, 1.0, -0.5), (0.75, 1.0, 0.0), (-0.0, 0.0, 0.0), (0.0, -0.0, 0.5),
    ]
    nc = len(cases)
    reps = (4 << 20) // (2 * 4 * 4 * nc) + 8
    b = nc * reps
    table = np.array([[e] * 4 for e, _, _ in cases], dtype=np.float64)
    q1 = np.tile(np.array([[c] * 4 for _, c, _ in cases], dtype=np.float64), (reps, 1))
    q2 = np.tile(np.array([[o] * 4 for _, _, o in cases], dtype=np.float64), (reps, 1))
    idx = np.tile(np.arange(nc, dtype=np.int64), reps)[:, None]            # query i meets entity i % nc
    gs = np.random.default_rng(3).integers(1, 4, (b, 1)).astype(np.float64)  # small integers: sums are exact
    params = fused.score_params(24.0, 0.5)
    t_table, t_q1, t_q2, t_gs = dev(table), dev(q1), dev(q2), dev(gs)
    t_idx = torch.tensor(idx, device="cuda")
    plan = fused.build_plan(t_idx, nc)
    score = fused.score_forward("box", t_table, t_idx, t_q1, t_q2, params)
    g_rows, g_c, g_o = orc.score_backward("box", gs, table[idx], q1[:, None], q2[:, None], 0.5)
    want = np.zeros((nc, 4))
    np.add.at(want, idx.reshape(-1), g_rows.reshape(-1, 4))
    saved = fused.new_codes("box", t_table, t_idx, t_q1)
    assert torch.equal(fused.score_forward("box", t_table, t_idx, t_q1, t_q2, params, codes=saved), score)
    for codes in (None, saved):   # codes made by the query-gradient kernel / by the forward
        merged = torch.empty((nc, 4), device="cuda")
        g1, g2 = fused.score_backward_fused("box", plan, t_table, t_idx, t_q1, t_q2, score, t_gs, params,
                                            merged=merged, codes=codes)
        assert np.array_equal(merged.cpu().numpy().astype(np.float64), want)
        assert np.array_equal(g1.cpu().numpy().astype(np.float64), g_c[:, 0])
        assert np.array_equal(g2.cpu().numpy().astype(np.float64), g_o[:, 0])


def test_sign_codes_are_refused_where_they_do_not_exist():
    from smore_amd import fused
    t = torch.zeros(10, 8, device="cuda")
    q = torch.zeros(2, 8, device="cuda")
    idx = torch.zeros(2, 3, dtype=torch.int64, device="cuda")
    assert fused.new_codes("l2", t, idx, q) is None
    assert fused.new_codes("box", torch.zeros(10, 2048, device="cuda"), idx, torch.zeros(2, 2048, device="cuda")) is None
    buf = torch.zeros(2 * 3 * 64, dtype=torch.uint8, device="cuda")
    with pytest.raises(Exception, match="no sign codes"):
        fused.score_forward("l2", t, idx, q, None, fused.score_params(1.0), codes=buf)
    with pytest.raises(Exception, match="smx_score_codes_bytes"):
        fused.score_forward("box", t, idx, q, q, fused.score_params(1.0), codes=buf[:64])


@pytest.mark.parametrize("kind", ["adam", "sgd", "adagrad", "rmsprop"])
@pytest.mark.parametrize("squeeze", [False, True])
def test_fused_entity_pass_with_every_optimizer(kind, squeeze):
    """Gather-fused entity backward + row update for each optimizer kind, long and short segments,
    both through the entity pass alone and through the one-call backward."""
    from smore_amd import fused
    rng = np.random.default_rng(21)
    n, b, k, dim, lr = 600, 24, 128, 48, 1e-2
    table, q1, q2, idx, gs = make_problem("box", n, b, k, dim, rng, zipf=1.2)
    t_q1, t_q2, t_gs = dev(q1), dev(q2), dev(gs)
    t_idx = torch.tensor(idx, device="cuda")
    params = fused.score_params(24.0, 0.02)
    plan = fused.build_plan(t_idx, n, want_inverse=True)
    uniq, inverse, _, _ = orc.merge_indices(idx)
    for one_call in (False, True):
        t_w = dev(table)
        t_m = torch.zeros_like(t_w) if kind == "adam" else None
        t_v = None if kind == "sgd" else (torch.zeros((n, 1), device="cuda") if squeeze else torch.zeros_like(t_w))
        w, m = table.copy(), np.zeros_like(table)
        v = np.zeros((n, 1)) if squeeze else np.zeros_like(table)
        for step in (1, 2):
            score = fused.score_forward("box", t_w, t_idx, t_q1, t_q2, params)
            merged = torch.empty((uniq.size, dim), device="cuda")
            fused.score_backward_entity("box", plan, t_w, t_q1, t_q2, score, t_gs, params, merged=merged)
            g = merged.cpu().numpy().astype(np.float64)  # the device's own merged gradient isolates the update rule
            w_s, m_s, v_s = t_w.cpu().numpy().astype(np.float64), None, None
            if t_m is not None:
                m_s = t_m.cpu().numpy().astype(np.float64)
            if t_v is not None:
                v_s = t_v.cpu().numpy().astype(np.float64)
            if kind == "adam":
                orc.adam_rows(w_s, m_s, v_s, uniq, g, lr, step, squeeze=squeeze)
            elif kind == "sgd":
                orc.sgd_rows(w_s, uniq, g, lr)
            elif kind == "adagrad":
                orc.adagrad_rows(w_s, v_s, uniq, g, lr, squeeze=squeeze)
            else:
                orc.rmsprop_rows(w_s, v_s, uniq, g, lr, squeeze=squeeze)
            op = fused.opt_params(kind, lr, step=step, squeeze=squeeze)
            if one_call:
                fused.score_backward_fused("box", plan, t_w, t_idx, t_q1, t_q2, score, t_gs, params, m=t_m, v=t_v, adam=op)
            else:
                fused.score_backward_entity("box", plan, t_w, t_q1, t_q2, score, t_gs, params, m=t_m, v=t_v, adam=op)
            assert_close(t_w.cpu().numpy(), w_s, REL_F32, f"{kind} w step {step}")
            if t_v is not None:
                assert_close(t_v.cpu().numpy(), v_s, REL_F32, f"{kind} v step {step}")
            if t_m is not None:
                assert_close(t_m.cpu().numpy(), m_s, REL_F32, f"{kind} m step {step}")


@pytest.mark.parametrize("shape", [
    (7, 1, 1, 4),        # a single pair
    (50, 9, 1, 16),      # K = 1: the positives layout [B,1]
    (50, 1, 333, 16),    # one query, ragged K
    (1, 5, 70, 8),       # a table of one row: one segment holds every pair
    (100000, 3, 65, 4),  # every id distinct with high probability: only one-pair segments
    (64, 2, 3, 2048),    # the widest row the fused path takes (8 float4 columns per lane)
    (64, 2, 3, 252),     # widest unaligned-friendly scalar row is 256; 252 is float4-aligned
    (30, 2, 5, 255),     # scalar columns, four per lane
    (40, 2, 70, 800),    # two-query models: eight wavefronts' rows + slabs would pass 64 KiB of LDS here
    (40, 2, 70, 848),
    (40, 2, 70, 1600),   # the same band for one-query models
    (40, 2, 70, 1704),
])
def test_fused_edge_shapes(shape):
    n, b, k, dim = shape
    run_case("box", n, b, k, dim, adam_steps=1)
    run_case("l2", n, b, k, dim, adam_steps=1)


def test_one_giant_segment_and_all_long_segments():
    """Every pair hits one of three ids: nothing but long segments, many tiles each."""
    from smore_amd import fused
    rng = np.random.default_rng(31)
    n, b, k, dim = 3, 40, 500, 32
    table, q1, q2, idx, gs = make_problem("rotate", n, b, k, dim, rng)
    t_table, t_q1, t_q2, t_gs = dev(table), dev(q1), dev(q2), dev(gs)
    t_idx = torch.tensor(idx, device="cuda")
    params = fused.score_params(9.0)
    plan = fused.build_plan(t_idx, n, want_inverse=True)
    assert plan.n_uniq == 3
    score = fused.score_forward("rotate", t_table, t_idx, t_q1, t_q2, params)
    merged = torch.empty((3, 2 * dim), device="cuda")
    fused.score_backward_entity("rotate", plan, t_table, t_q1, t_q2, score, t_gs, params, merged=merged)
    rows = orc.gather(table, idx).reshape(b, k, -1)
    g_rows, _, _ = orc.score_backward("rotate", gs, rows, q1[:, None], q2[:, None])
    uniq, inverse, _, _ = orc.merge_indices(idx)
    want = orc.merge_grads(g_rows.reshape(b * k, -1), inverse, 3)
    sum_abs = orc.merge_grads(np.abs(g_rows).reshape(b * k, -1), inverse, 3)
    assert_close(merged.cpu().numpy(), want, REL_F32, "giant segments", sum_abs=sum_abs)


def test_unsupported_rows_are_refused_not_mangled():
    from smore_amd import _lib, fused
    idx = torch.zeros(2, 3, dtype=torch.int64, device="cuda")
    for dim in (2052, 257):  # too wide for float4 columns / for scalar columns
        t = torch.zeros(10, dim, device="cuda")
        q = torch.zeros(2, dim, device="cuda")
        with pytest.raises(_lib.SmxError):
            fused.score_forward("l1", t, idx, q, None, fused.score_params(1.0))
    with pytest.raises(_lib.SmxError):  # regulariser prologue is a BetaE feature
        fused.score_forward("l1", torch.zeros(10, 8, device="cuda"), idx, torch.zeros(2, 8, device="cuda"), None,
                            fused.score_params(1.0, regularizer=(1.0, 0.05, 1e9)))
    with pytest.raises(_lib.SmxError):  # empty batch
        fused.build_plan(torch.zeros(0, dtype=torch.int64, device="cuda"), 10)


def test_second_stream_backward_gives_the_bits_of_the_serial_one():
    """Steps of a million pairs or more with the forward's codes and an optimizer run the entity pass on
    the library's second stream beside the query-gradient kernel.  Same kernels, same data, disjoint
    rows: the results must be bit-identical to the one-stream order, and repeatable."""
    import bench
    from smore_amd import fused
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7)
    n, b, k, dim = 2_000_000, 1100, 1024, 200
    table = torch.empty((n, dim), device="cuda").uniform_(-0.07, 0.07, generator=gen)
    q1 = torch.empty((b, dim), device="cuda").uniform_(-0.07, 0.07, generator=gen)
    q2 = torch.empty((b, dim), device="cuda").uniform_(0.0, 0.07, generator=gen)
    idx = bench.zipf_ids(n, (b, k), 1.1, gen, torch.device("cuda"))
    gs = torch.randn((b, k), device="cuda", generator=gen)
    params = fused.score_params(24.0, 0.02)
    plan = fused.build_plan(idx, n)
    codes = fused.new_codes("box", table, idx, q1)
    score = fused.score_forward("box", table, idx, q1, q2, params, codes=codes)
    results = []
    for serial in (1, 0, 0):
        _serial_backward(serial)
        w, m, v = table.clone(), torch.zeros_like(table), torch.zeros_like(table)
        g1, g2 = fused.score_backward_fused("box", plan, w, idx, q1, q2, score, gs, params, m=m, v=v,
                                            adam=fused.adam_params(1e-4, 1), codes=codes)
        torch.cuda.synchronize()
        results.append((g1, g2, w, m, v))
    for other in results[1:]:
        for a, c in zip(results[0], other):
            assert torch.equal(a, c)
    touched = (results[0][3].abs().sum(dim=1) != 0).sum().item()
    assert abs(touched - plan.n_uniq) <= int((gs == 0).sum().item())


def test_deferred_entity_pass_matches_the_one_call_backward():
    """The autograd flow takes the query gradients first and updates the rows later, in
    score_backward_entity.  For large steps with the forward's codes that call hands the one-pair
    segments to the pair-ordered kernel and runs the entity pass beside it: table, m and v must come
    out bit-identical to the one-call backward and to the one-stream order."""
    import bench
    from smore_amd import fused
    gen = torch.Generator(device="cuda")
    gen.manual_seed(11)
    n, b, k, dim = 1_500_000, 2800, 384, 200          # queries 4.5 MB (> one L2), 1.07 M pairs
    table = torch.empty((n, dim), device="cuda").uniform_(-0.07, 0.07, generator=gen)
    q1 = torch.empty((b, dim), device="cuda").uniform_(-0.07, 0.07, generator=gen)
    q2 = torch.empty((b, dim), device="cuda").uniform_(0.0, 0.07, generator=gen)
    idx = bench.zipf_ids(n, (b, k), 1.1, gen, torch.device("cuda"))
    gs = torch.randn((b, k), device="cuda", generator=gen)
    params = fused.score_params(24.0, 0.02)
    plan = fused.build_plan(idx, n)
    codes = fused.new_codes("box", table, idx, q1)
    score = fused.score_forward("box", table, idx, q1, q2, params, codes=codes)
    for squeeze in (False, True):
        def state():
            v_shape = (n, 1) if squeeze else (n, dim)
            return table.clone(), torch.zeros_like(table), torch.zeros(v_shape, device="cuda")
        opt = fused.adam_params(1e-4, 1, squeeze=squeeze)
        _serial_backward(0)
        w0, m0, v0 = state()
        g1, g2 = fused.score_backward_fused("box", plan, w0, idx, q1, q2, score, gs, params, m=m0, v=v0, adam=opt,
                                            codes=codes)
        outcomes = []
        for serial in (0, 1, 0):
            _serial_backward(serial)
            w, m, v = state()
            d1, d2 = fused.score_backward_query("box", table, idx, q1, q2, score, gs, params, codes=codes)
            fused.score_backward_entity("box", plan, w, q1, q2, score, gs, params, m=m, v=v, adam=opt, codes=codes)
            torch.cuda.synchronize()
            outcomes.append((d1, d2, w, m, v))
        for got in outcomes:
            for a, c, what in zip((g1, g2, w0, m0, v0), got, ("gq1", "gq2", "table", "m", "v")):
                assert torch.equal(a, c), (what, squeeze)
        assert (m0.abs().sum(dim=1) != 0).sum().item() > 0.9 * plan.n_uniq


@pytest.mark.parametrize("b,k,dim", [(6, 50, 128), (3, 7, 30), (40, 300, 200)])
def test_l1_sign_codes(b, k, dim):
    """L1 keeps one decision per feature (e - q > 0, ties go to -1): forward-saved codes, codes written by the
    query-gradient kernel, and the recomputing path give the same merged rows bit for bit; ties included."""
    from smore_amd import fused
    rng = np.random.default_rng(k)
    n = 40
    table, q1, _, idx, gs = make_problem("l1", n, b, k, dim, rng)
    table[3] = q1[0]                      # exact ties: entity 3 equals query 0 ...
    idx[0, :3] = 3                        # ... and they meet
    t_table, t_q1, t_gs = dev(table), dev(q1), dev(gs)
    t_idx = torch.tensor(idx, device="cuda")
    params = fused.score_params(12.0)
    plan = fused.build_plan(t_idx, n)
    saved = fused.new_codes("l1", t_table, t_idx, t_q1)
    assert saved is not None
    score = fused.score_forward("l1", t_table, t_idx, t_q1, None, params, codes=saved)
    assert torch.equal(score, fused.score_forward("l1", t_table, t_idx, t_q1, None, params))
    out = {}
    for how in ("recompute", "forward"):
        merged = torch.full((plan.n_uniq, dim), float("nan"), device="cuda")
        g1, _ = fused.score_backward_fused("l1", plan, t_table, t_idx, t_q1, None, score, t_gs, params, merged=merged,
                                           sign_codes=False, codes=saved if how == "forward" else None)
        out[how] = (merged.cpu().numpy(), g1.cpu().numpy())
    assert np.array_equal(out["forward"][0], out["recompute"][0])
    assert_close(out["forward"][1], out["recompute"][1], 1e-6, "gq1")
    g_rows, g_q, _ = orc.score_backward("l1", gs, table[idx], q1[:, None], None, 0.0)
    uniq, inv = np.unique(idx.reshape(-1), return_inverse=True)
    want = np.zeros((len(uniq), dim))
    np.add.at(want, inv, g_rows.reshape(-1, dim))
    sum_abs = np.zeros((len(uniq), dim))
    np.add.at(sum_abs, inv, np.abs(g_rows.reshape(-1, dim)))
    assert_close(out["forward"][0], want, REL_F32, "merged vs oracle", sum_abs=sum_abs)
    assert_close(out["forward"][1], g_q[:, 0], REL_F32, "gq1 vs oracle")


def test_l1_codes_written_by_the_query_gradient_kernel():
    """More than 4 MiB of L1 queries: without forward codes the one-call backward writes the codes itself
    for the entity pass; merged rows must equal the recomputing path's bit for bit."""
    from smore_amd import fused
    rng = np.random.default_rng(2)
    n, b, k, dim = 500, 8300, 3, 128
    table, q1, _, idx, gs = make_problem("l1", n, b, k, dim, rng, zipf=1.1)
    t_table, t_q1, t_gs = dev(table), dev(q1), dev(gs)
    t_idx = torch.tensor(idx, device="cuda")
    params = fused.score_params(12.0)
    plan = fused.build_plan(t_idx, n)
    score = fused.score_forward("l1", t_table, t_idx, t_q1, None, params)
    out = []
    for codes in (False, True):
        merged = torch.full((plan.n_uniq, dim), float("nan"), device="cuda")
        g1, _ = fused.score_backward_fused("l1", plan, t_table, t_idx, t_q1, None, score, t_gs, params, merged=merged,
                                           sign_codes=codes)
        out.append((merged.cpu().numpy(), g1.cpu().numpy()))
    assert np.array_equal(out[0][0], out[1][0])
    assert_close(out[1][1], out[0][1], 1e-6, "gq1")


@pytest.mark.parametrize("model", ["box", "l1", "l2", "rotate", "beta_kl", "complex", "distmult"])
def test_entity_pass_over_several_index_streams(model):
    """smx_score_backward_entity_multi: three index streams of one query batch (K = 1, 7, 20; the first is what a
    positive lookup looks like) behind one plan.  Merged rows against the oracle's unique-merge + scatter-sum over
    the concatenated streams (embed_optimizer.py:39-48,155-163), then one Adam step per entity."""
    from smore_amd import fused
    n, b, dim, ks, lr = 150, 9, 24, (1, 7, 20), 1e-3
    rng = np.random.default_rng(seed("multi", model))
    table, q1, q2, _, _ = make_problem(model, n, b, 1, dim, rng)
    gamma, cen = GAMMA[model], 0.02
    params = fused.score_params(gamma, cen)
    t_table, t_q1, t_q2 = dev(table), dev(q1), dev(q2)
    o_q1 = q1[:, None, :]
    o_q2 = None if q2 is None else q2[:, None, :]
    ids, sources, o_rows = [], [], []
    for k in ks:
        idx = rng.integers(0, n, (b, k))
        idx[0, 0] = 5                                   # an entity present in every stream
        gs = rng.standard_normal((b, k)).astype(np.float32).astype(np.float64)
        t_idx = torch.tensor(idx, device="cuda")
        codes = fused.new_codes(model, t_table, t_idx, t_q1)
        score = fused.score_forward(model, t_table, t_idx, t_q1, t_q2, params, codes=codes)
        sources.append((score, dev(gs), codes))
        ids.append(idx)
        rows = orc.gather(table, idx).reshape(b, k, -1)
        g_rows, _, _ = orc.score_backward(model, gs, rows, o_q1, o_q2, cen)
        o_rows.append(g_rows.reshape(b * k, -1))
    flat = np.concatenate([i.reshape(-1) for i in ids])
    plan = fused.build_plan(torch.tensor(flat, device="cuda"), n, want_inverse=True)
    uniq, inverse, _, _ = orc.merge_indices(flat)
    o_merged = orc.merge_grads(np.concatenate(o_rows), inverse, uniq.size)
    o_abs = orc.merge_grads(np.abs(np.concatenate(o_rows)), inverse, uniq.size)
    merged = torch.full((uniq.size, table.shape[1]), float("nan"), device="cuda")
    fused.score_backward_entity_multi(model, plan, t_table, t_q1, t_q2, sources, params, merged=merged)
    assert_close(merged.cpu().numpy(), o_merged, REL_F32, f"{model} merged over three streams", sum_abs=o_abs)
    # the optimizer step from the same pass, checked from the device's own merged rows
    t_m, t_v = torch.zeros_like(t_table), torch.zeros_like(t_table)
    w_s, m_s, v_s = table.copy(), np.zeros_like(table), np.zeros_like(table)
    orc.adam_rows(w_s, m_s, v_s, uniq, merged.cpu().numpy().astype(np.float64), lr, 1)
    fused.score_backward_entity_multi(model, plan, t_table, t_q1, t_q2, sources, params, m=t_m, v=t_v,
                                      adam=fused.adam_params(lr, 1))
    touched = np.zeros(n, bool)
    touched[uniq] = True
    assert_close(t_table.cpu().numpy()[touched], w_s[touched], REL_F32, f"{model} w over three streams")
    assert_close(t_m.cpu().numpy()[touched], m_s[touched], REL_F32, f"{model} m over three streams")
    assert_close(t_v.cpu().numpy()[touched], v_s[touched], REL_F32, f"{model} v over three streams", rms_floor=False)
    assert np.array_equal(t_table.cpu().numpy()[~touched], table[~touched].astype(np.float32))
    # one source through the same entry point is the single-stream call
    one = torch.full((plan.n_uniq, table.shape[1]), float("nan"), device="cuda")
    t_idx = torch.tensor(ids[2], device="cuda")
    plan1 = fused.build_plan(t_idx, n)
    a = torch.full((plan1.n_uniq, table.shape[1]), float("nan"), device="cuda")
    b_ = torch.full_like(a, float("nan"))
    fused.score_backward_entity_multi(model, plan1, dev(table), t_q1, t_q2, sources[2:], params, merged=a)
    fused.score_backward_entity(model, plan1, dev(table), t_q1, t_q2, sources[2][0], sources[2][1], params, merged=b_,
                                codes=sources[2][2])
    assert torch.equal(a, b_)


@pytest.mark.parametrize("model", ["box", "l1", "l2", "rotate", "beta_kl", "distmult"])
def test_entity_pass_over_streams_of_different_query_batches(model, shapes=((5, 7), (3, 20), (8, 1)), dim=24, n=120):
    """Records of several forward calls in one step (the reference merges them like any others,
    embed_optimizer.py:155-163): three streams of three query batches (B = 5, 3, 8; K = 7, 20, 1) whose query rows lie
    one after the other, each source naming its stretch; the second and third batch share entities with the first.
    Merged rows against the oracle's unique-merge + scatter-sum, then one Adam step."""
    from smore_amd import fused
    lr = 1e-3
    rng = np.random.default_rng(seed("multi-batch", model, dim, n, *[x for s in shapes for x in s]))
    b_all = sum(b for b, _ in shapes)
    table, q1, q2, _, _ = make_problem(model, n, b_all, 1, dim, rng)
    gamma, cen = GAMMA[model], 0.02
    params = fused.score_params(gamma, cen)
    t_table, t_q1, t_q2 = dev(table), dev(q1), dev(q2)
    ids, sources, o_rows, at = [], [], [], 0
    for b, k in shapes:
        idx = rng.integers(0, n, (b, k))
        idx[0, 0] = min(5, n - 1)                       # an entity present in every stream
        gs = rng.standard_normal((b, k)).astype(np.float32).astype(np.float64)
        t_idx = torch.tensor(idx, device="cuda")
        s_q1 = t_q1[at:at + b]
        s_q2 = None if t_q2 is None else t_q2[at:at + b]
        codes = fused.new_codes(model, t_table, t_idx, s_q1)
        score = fused.score_forward(model, t_table, t_idx, s_q1, s_q2, params, codes=codes)
        sources.append((score, dev(gs), codes, None, at, b))
        ids.append(idx)
        rows = orc.gather(table, idx).reshape(b, k, -1)
        g_rows, _, _ = orc.score_backward(model, gs, rows, q1[at:at + b, None, :],
                                          None if q2 is None else q2[at:at + b, None, :], cen)
        o_rows.append(g_rows.reshape(b * k, -1))
        at += b
    flat = np.concatenate([i.reshape(-1) for i in ids])
    plan = fused.build_plan(torch.tensor(flat, device="cuda"), n, want_inverse=True)
    uniq, inverse, _, _ = orc.merge_indices(flat)
    o_merged = orc.merge_grads(np.concatenate(o_rows), inverse, uniq.size)
    o_abs = orc.merge_grads(np.abs(np.concatenate(o_rows)), inverse, uniq.size)
    merged = torch.full((uniq.size, table.shape[1]), float("nan"), device="cuda")
    fused.score_backward_entity_multi(model, plan, t_table, t_q1, t_q2, sources, params, merged=merged)
    assert_close(merged.cpu().numpy(), o_merged, REL_F32, f"{model} merged over three query batches", sum_abs=o_abs)
    t_m, t_v = torch.zeros_like(t_table), torch.zeros_like(t_table)
    w_s, m_s, v_s = table.copy(), np.zeros_like(table), np.zeros_like(table)
    orc.adam_rows(w_s, m_s, v_s, uniq, merged.cpu().numpy().astype(np.float64), lr, 1)
    fused.score_backward_entity_multi(model, plan, t_table, t_q1, t_q2, sources, params, m=t_m, v=t_v,
                                      adam=fused.adam_params(lr, 1))
    touched = np.zeros(n, bool)
    touched[uniq] = True
    assert_close(t_table.cpu().numpy()[touched], w_s[touched], REL_F32, f"{model} w over three query batches")
    assert_close(t_m.cpu().numpy()[touched], m_s[touched], REL_F32, f"{model} m over three query batches")
    assert np.array_equal(t_table.cpu().numpy()[~touched], table[~touched].astype(np.float32))
    # a stretch of queries that does not exist is refused
    bad = list(sources)
    bad[-1] = sources[-1][:4] + (b_all - shapes[-1][0] + 1, shapes[-1][0])
    with pytest.raises(Exception):
        fused.score_backward_entity_multi(model, plan, t_table, t_q1, t_q2, bad, params, merged=merged)


def test_several_index_streams_at_a_size_that_forks():
    """Two streams (K = 1 and 300) of 4096 box queries, Adam: more than a million pairs and queries beyond one L2,
    so ids that occur once go through the pair-ordered kernel (one launch per stream) beside the entity pass.
    Against the same pairs laid out as one [B, 301] stream: the same rows are touched, the same values up to the
    order of summation."""
    from smore_amd import fused
    n, b, dim, lr = 400_000, 4096, 200, 1e-3
    g = torch.Generator(device="cuda").manual_seed(3)
    table = torch.empty((n, dim), device="cuda").uniform_(-0.07, 0.07, generator=g)
    q1 = torch.empty((b, dim), device="cuda").uniform_(-0.07, 0.07, generator=g)
    q2 = torch.empty((b, dim), device="cuda").uniform_(-0.07, 0.07, generator=g).abs_()
    pos = torch.randint(0, n, (b, 1), device="cuda", generator=g)
    neg = torch.randint(0, n, (b, 300), device="cuda", generator=g)
    gp = torch.randn((b, 1), device="cuda", generator=g)
    gn = torch.randn((b, 300), device="cuda", generator=g)
    params = fused.score_params(24.0, 0.02)

    def run(streams, batches=False):
        w, m, v = table.clone(), torch.zeros_like(table), torch.zeros_like(table)
        sources = []
        for i, (ids, gs) in enumerate(streams):
            codes = fused.new_codes("box", w, ids, q1)
            assert codes is not None
            src = (fused.score_forward("box", w, ids, q1, q2, params, codes=codes), gs.contiguous(), codes)
            # batches: every stream has a query batch of its own (here: copies), the later stream's rows first
            sources.append(src + (None, (len(streams) - 1 - i) * b, b) if batches else src)
        plan = fused.build_plan(torch.cat([ids.reshape(-1) for ids, _ in streams]), n)
        reps = len(streams) if batches else 1
        fused.score_backward_entity_multi("box", plan, w, q1.repeat(reps, 1), q2.repeat(reps, 1), sources, params, m=m,
                                          v=v, adam=fused.adam_params(lr, 1))
        return w, m, v, plan

    w2, m2, v2, plan2 = run([(pos, gp), (neg, gn)])
    w3, m3, v3, _ = run([(pos, gp), (neg, gn)], batches=True)
    assert torch.equal(w3, w2) and torch.equal(m3, m2) and torch.equal(v3, v2), "a query batch per stream: the same bits"
    w1, m1, v1, plan1 = run([(torch.cat([pos, neg], dim=1), torch.cat([gp, gn], dim=1))])
    assert plan1.n_uniq == plan2.n_uniq and torch.equal(plan1.uniq, plan2.uniq)
    assert (plan2.pair_seg < 0).sum().item() > 30_000, "the case must have one-pair ids"
    touched = torch.zeros(n, dtype=torch.bool, device="cuda")
    touched[plan2.uniq] = True
    assert torch.equal(w2[~touched], table[~touched]) and not bool(m2[~touched].any())
    assert_close(m2[touched].cpu().numpy(), m1[touched].cpu().numpy(), REL_F32, "m, two streams vs one")
    assert_close(v2[touched].cpu().numpy(), v1[touched].cpu().numpy(), REL_F32, "v, two streams vs one")
    assert float((w2 - w1).abs().max()) <= 2 * lr
    assert float(((w2 - w1).abs() > 1e-5 * 0.07).float().mean()) < 1e-4


@pytest.mark.parametrize("model,dim", [("box", 200), ("box", 400), ("l1", 30), ("l2", 64), ("rotate", 48), ("beta_kl", 20)])
def test_forward_scores_each_distinct_entity_of_a_tile_once(model, dim):
    """The forward de-duplicates ids inside a workgroup's tile of negatives: every pair must still get
    the bits it would get alone.  Queries whose negatives are all one entity, all distinct, drawn from three
    entities, and a last batch of 6 pairs (K = 70); scores against the dense layout (rows given pair by pair, no
    ids, no de-duplication) bit for bit and against the oracle; sign codes (box, l1) through the backward that
    reads them against the backward that recomputes from the rows, bit for bit."""
    from smore_amd import fused
    rng = np.random.default_rng(seed("dedup", model, dim))
    n, b, k = 90, 5, 70
    table, q1, q2, idx, gs = make_problem(model, n, b, k, dim, rng)
    idx[0, :] = 7
    idx[1, :] = np.arange(k) % n
    idx[2, :] = rng.choice([3, 4, 88], size=k)
    idx[3, :64] = 11                                   # the first batch all equal, the short last batch distinct
    idx[3, 64:] = np.arange(6) + 20
    gamma = GAMMA[model]
    params = fused.score_params(gamma, 0.02)
    t_table, t_q1, t_q2, t_gs = dev(table), dev(q1), dev(q2), dev(gs)
    t_idx = torch.tensor(idx, device="cuda")
    score = fused.score_forward(model, t_table, t_idx, t_q1, t_q2, params)
    rows = orc.gather(table, idx).reshape(b, k, -1)
    dense = fused.score_forward(model, dev(rows.reshape(b * k, -1)), None, t_q1, t_q2, params)
    assert torch.equal(score, dense)
    want = orc.score_forward(model, rows, q1[:, None], None if q2 is None else q2[:, None], gamma, 0.02)
    assert_close(score.cpu().numpy(), want, REL_F32, f"{model} score with repeated ids", rms_floor=model == "beta_kl")
    assert bool((score[0] == score[0, 0]).all()) and bool((score[3, :64] == score[3, 0]).all())
    codes = fused.new_codes(model, t_table, t_idx, t_q1)
    if model in ("box", "l1"):
        assert codes is not None
        score_c = fused.score_forward(model, t_table, t_idx, t_q1, t_q2, params, codes=codes)
        assert torch.equal(score_c, score)
        per_pair = codes.view(b, k, -1)
        assert torch.equal(per_pair[0], per_pair[0, :1].expand(k, -1)), "repeats must carry their representative's codes"
        plan = fused.build_plan(t_idx, n)
        got = {}
        for use in (True, False):
            merged = torch.full((plan.n_uniq, table.shape[1]), float("nan"), device="cuda")
            g1, g2 = fused.score_backward_fused(model, plan, t_table, t_idx, t_q1, t_q2, score, t_gs, params,
                                                merged=merged, sign_codes=False, codes=codes if use else None)
            got[use] = (merged, g1, g2)
        assert torch.equal(got[True][0], got[False][0])
        assert_close(got[True][1].cpu().numpy(), got[False][1].cpu().numpy(), 1e-6, "gq1 from the forward's codes")
    else:
        assert codes is None


@pytest.mark.parametrize("model,dim,n", [("box", 16, 3000), ("l2", 8, 200), ("box", 200, 100_000), ("rotate", 24, 700)])
def test_forward_de_duplication_over_full_tiles(model, dim, n):
    """2 M pairs, so that the forward takes tiles of 256 negatives (four wavefronts share one hash table and one list
    of distinct entities): skewed ids from a small table -- every tile holds repeats inside and across its
    wavefronts, and ids that collide in the table's slots.  Scores against the dense layout (rows given pair by pair,
    nothing to de-duplicate) bit for bit; the sign codes of repeats must be their representative's; the
    query gradient from those codes against the recomputing backward."""
    from smore_amd import fused
    rng = np.random.default_rng(seed("dedup-tiles", model, dim, n))
    b, k = 2048, 1024
    table = rng.uniform(-0.07, 0.07, (n, dim * (2 if model == "rotate" else 1))).astype(np.float32)
    q1 = rng.uniform(-0.07, 0.07, (b, dim)).astype(np.float32)
    q2 = np.abs(rng.uniform(-0.07, 0.07, (b, dim))).astype(np.float32) if model in ("box", "rotate") else None
    idx = np.minimum((rng.pareto(0.9, (b, k)) * 3).astype(np.int64), n - 1)
    idx[5, :] = 17                                     # a query whose negatives are one entity
    idx[6, :] = (np.arange(k) * 7) % n                 # ... and one without repeats inside a tile
    t_table, t_q1, t_q2 = torch.tensor(table, device="cuda"), torch.tensor(q1, device="cuda"), None if q2 is None else torch.tensor(q2, device="cuda")
    t_idx = torch.tensor(idx, device="cuda")
    params = fused.score_params(GAMMA[model], 0.02)
    err = fused.new_error_flag("cuda")
    score = fused.score_forward(model, t_table, t_idx, t_q1, t_q2, params, err)
    dense = torch.empty_like(score)
    for b0 in range(0, b, 256):                        # the dense layout in slices: [256 * K, dim] rows at a time
        rows = t_table[t_idx[b0:b0 + 256].reshape(-1)]
        dense[b0:b0 + 256] = fused.score_forward(model, rows, None, t_q1[b0:b0 + 256], None if t_q2 is None else t_q2[b0:b0 + 256], params)
    if model in ("box", "l1"):
        assert torch.equal(score, dense)
    else:   # a row's multiply-adds may be contracted differently where it stands in a wavefront's stream
        assert_close(score.cpu().numpy(), dense.cpu().numpy(), 2e-6, f"{model} forward over full tiles vs the dense layout")
    assert err.item() == 0
    for _ in range(3):   # which wavefront scores which row is fixed: the same bits in every run
        assert torch.equal(fused.score_forward(model, t_table, t_idx, t_q1, t_q2, params, err), score)
    codes = fused.new_codes(model, t_table, t_idx, t_q1)
    if codes is not None:
        score_c = fused.score_forward(model, t_table, t_idx, t_q1, t_q2, params, codes=codes)
        assert torch.equal(score_c, score)
        per_pair = codes.view(b, k, -1)
        assert torch.equal(per_pair[5], per_pair[5, :1].expand(k, -1)), "repeats must carry their representative's codes"
        same = t_idx[:64, 1:] == t_idx[:64, :-1]       # neighbours with one id: one code record
        assert torch.equal(per_pair[:64, 1:][same], per_pair[:64, :-1][same])
        gs = torch.randn((b, k), device="cuda", generator=torch.Generator(device="cuda").manual_seed(3))
        from_codes = fused.score_backward_query(model, t_table, t_idx, t_q1, t_q2, score, gs, params, codes=codes)
        recomputed = fused.score_backward_query(model, t_table, t_idx, t_q1, t_q2, score, gs, params)
        assert_close(from_codes[0].cpu().numpy(), recomputed[0].cpu().numpy(), 1e-6, "gq1 from the forward's codes, full tiles")


@pytest.mark.parametrize("model,ks,dim", [("box", (12,), 24), ("box", (1, 20), 24), ("l1", (1, 7), 24), ("l2", (5,), 24),
                                          ("rotate", (1, 9), 24), ("beta_kl", (1, 6), 24), ("complex", (4,), 24),
                                          ("distmult", (1, 3), 24),
                                          # single-float columns, and rows of several column groups per lane
                                          ("l1", (1, 7), 30), ("box", (3,), 520), ("rotate", (2,), 130), ("box", (1, 4), 200),
                                          # rows too long for the fix-up kernel's wavefronts to share the lookup rows
                                          ("rotate", (2,), 600)])
def test_entity_pass_with_gradient_rows_of_plain_lookups(model, ks, dim):
    """The step's plain lookups (anchor entities, models/box.py:137) hand the optimizer materialised gradient rows
    (embed_optimizer.py:63-66); they go behind the fused streams in one plan, and an entity named by both gets one
    update from the sum (embed_optimizer.py:155-163).  Rows for ids the streams also hold, for ids only the lookup
    holds, an id looked up 3 times, and one looked up 150 times (a segment longer than a tile, finished by the
    fix-up kernel).  Merged rows and the Adam step against the oracle's merge of the concatenation."""
    from smore_amd import fused
    n, b, lr = 700, 9, 1e-3
    rng = np.random.default_rng(seed("plain lookups", model, ks, dim))
    table, q1, q2, _, _ = make_problem(model, n, b, 1, dim, rng)
    gamma, cen = GAMMA[model], 0.02
    params = fused.score_params(gamma, cen)
    t_table, t_q1, t_q2 = dev(table), dev(q1), dev(q2)
    o_q1 = q1[:, None, :]
    o_q2 = None if q2 is None else q2[:, None, :]
    ids, sources, o_rows = [], [], []
    for k in ks:
        idx = rng.integers(0, n // 2, (b, k))             # the upper half of the table is the lookup's alone
        idx[0, 0] = 5
        gs = rng.standard_normal((b, k)).astype(np.float32).astype(np.float64)
        t_idx = torch.tensor(idx, device="cuda")
        codes = fused.new_codes(model, t_table, t_idx, t_q1)
        score = fused.score_forward(model, t_table, t_idx, t_q1, t_q2, params, codes=codes)
        sources.append((score, dev(gs), codes))
        ids.append(idx.reshape(-1))
        rows = orc.gather(table, idx).reshape(b, k, -1)
        g_rows, _, _ = orc.score_backward(model, gs, rows, o_q1, o_q2, cen)
        o_rows.append(g_rows.reshape(b * k, -1))
    in_streams = np.unique(np.concatenate(ids))
    looked_up = np.concatenate([in_streams[:6], [5, 5, 5], rng.integers(n // 2, n, 10), np.full(150, 17),
                                np.full(150, n - 1)])
    rng.shuffle(looked_up)
    extra = rng.standard_normal((looked_up.size, table.shape[1])).astype(np.float32).astype(np.float64)
    flat = np.concatenate(ids + [looked_up])
    plan = fused.build_plan(torch.tensor(flat, device="cuda"), n, want_inverse=True)
    uniq, inverse, _, _ = orc.merge_indices(flat)
    all_rows = np.concatenate(o_rows + [extra])
    o_merged = orc.merge_grads(all_rows, inverse, uniq.size)
    o_abs = orc.merge_grads(np.abs(all_rows), inverse, uniq.size)
    merged = torch.full((uniq.size, table.shape[1]), float("nan"), device="cuda")
    fused.score_backward_entity_multi(model, plan, t_table, t_q1, t_q2, sources, params, merged=merged,
                                      grad_rows=dev(extra))
    assert_close(merged.cpu().numpy(), o_merged, REL_F32, f"{model} merged, streams + lookup rows", sum_abs=o_abs)
    t_m, t_v = torch.zeros_like(t_table), torch.zeros_like(t_table)
    w_s, m_s, v_s = table.copy(), np.zeros_like(table), np.zeros_like(table)
    orc.adam_rows(w_s, m_s, v_s, uniq, merged.cpu().numpy().astype(np.float64), lr, 1)
    fused.score_backward_entity_multi(model, plan, t_table, t_q1, t_q2, sources, params, m=t_m, v=t_v,
                                      adam=fused.adam_params(lr, 1), grad_rows=dev(extra))
    touched = np.zeros(n, bool)
    touched[uniq] = True
    assert touched[n - 1] and touched[17]
    assert_close(t_table.cpu().numpy()[touched], w_s[touched], REL_F32, f"{model} w, streams + lookup rows")
    assert_close(t_m.cpu().numpy()[touched], m_s[touched], REL_F32, f"{model} m, streams + lookup rows")
    assert_close(t_v.cpu().numpy()[touched], v_s[touched], REL_F32, f"{model} v, streams + lookup rows", rms_floor=False)
    assert np.array_equal(t_table.cpu().numpy()[~touched], table[~touched].astype(np.float32))


def test_gradient_rows_pass_the_clamp_mask_of_the_entity_prologue():
    """BetaE's prologue clamp(x + 1, 0.05, 1e9) masks the MODEL's gradient where the clamp is active
    (models/beta.py regularizer); the rows of a plain lookup are gradients with respect to the stored values
    already and are added after the mask."""
    from smore_amd import fused
    rng = np.random.default_rng(78)
    n, b, k, dim = 300, 6, 20, 24
    raw = (rng.standard_normal((n, 2 * dim)) * 1.5).astype(np.float32).astype(np.float64)
    f = lambda *s: np.clip(1 + rng.standard_normal(s), 0.05, 1e9).astype(np.float32).astype(np.float64)
    qa, qb = f(b, dim), f(b, dim)
    idx = rng.integers(0, n, (b, k))
    gs = rng.standard_normal((b, k)).astype(np.float32).astype(np.float64)
    params = fused.score_params(60.0, 0.0, regularizer=(1.0, 0.05, 1e9))
    t_raw, t_qa, t_qb = dev(raw), dev(qa), dev(qb)
    t_idx = torch.tensor(idx, device="cuda")
    score = fused.score_forward("beta_kl", t_raw, t_idx, t_qa, t_qb, params)
    rows = orc.gather(orc.regularizer(raw), idx).reshape(b, k, -1)
    g_rows, _, _ = orc.score_backward("beta_kl", gs, rows, qa[:, None], qb[:, None])
    looked_up = np.concatenate([idx[0, :5], idx[1, :3], [idx[0, 0]] * 2])
    extra = rng.standard_normal((looked_up.size, 2 * dim)).astype(np.float32).astype(np.float64)
    flat = np.concatenate([idx.reshape(-1), looked_up])
    plan = fused.build_plan(torch.tensor(flat, device="cuda"), n, want_inverse=True)
    uniq, inverse, _, _ = orc.merge_indices(flat)
    mask = ((raw + 1 >= 0.05) & (raw + 1 <= 1e9))
    assert not mask[looked_up].all(), "the looked-up rows must hit the clamp somewhere"
    model_rows = g_rows.reshape(b * k, -1) * mask[idx.reshape(-1)]
    o_merged = orc.merge_grads(np.concatenate([model_rows, extra]), inverse, uniq.size)
    merged = torch.empty((uniq.size, 2 * dim), device="cuda")
    fused.score_backward_entity_multi("beta_kl", plan, t_raw, t_qa, t_qb, [(score, dev(gs), None)], params,
                                      merged=merged, grad_rows=dev(extra))
    assert_close(merged.cpu().numpy(), o_merged, REL_F32, "masked model gradient + unmasked lookup rows")


@pytest.mark.parametrize("kind,squeeze", [("adam", True), ("sgd", False), ("adagrad", False), ("adagrad", True),
                                          ("rmsprop", False)])
def test_gradient_rows_reach_every_row_optimizer(kind, squeeze):
    """The rows of plain lookups are part of the gradient every optimizer of embed_optimizer.py sees (SGD :166-178,
    RMSprop :255-309, AdaGrad :312-349, Adam with the squeezed second moment :226-229): the update from the fused
    pass must equal the update from the materialised route (merged rows of the same call -> smx_rows_backward)."""
    from smore_amd import fused
    n, b, k, dim, lr = 400, 8, 16, 64, 1e-2
    rng = np.random.default_rng(seed("rows and optimizers", kind, squeeze))
    table, q1, q2, idx, gs = make_problem("box", n, b, k, dim, rng)
    params = fused.score_params(24.0, 0.02)
    t_q1, t_q2 = dev(q1), dev(q2)
    looked_up = np.concatenate([idx[0, :4], rng.integers(0, n, 12), np.full(70, int(idx[1, 0]))])
    extra = dev(rng.standard_normal((looked_up.size, dim)))
    flat = torch.tensor(np.concatenate([idx.reshape(-1), looked_up]), device="cuda")
    plan = fused.build_plan(flat, n)
    uniq_plan = fused.build_plan(plan.uniq, n)                      # the merged rows as one gradient row per entity
    out = {}
    for route in ("fused", "rows"):
        w = dev(table)
        m = torch.zeros_like(w) if kind == "adam" else None
        v = None if kind == "sgd" else (torch.full((n,), 0.01, device="cuda") if squeeze else torch.full_like(w, 0.01))
        t_idx = torch.tensor(idx, device="cuda")
        codes = fused.new_codes("box", w, t_idx, t_q1)
        score = fused.score_forward("box", w, t_idx, t_q1, t_q2, params, codes=codes)
        opt = fused.opt_params(kind, lr, step=3, squeeze=squeeze)
        if route == "fused":
            fused.score_backward_entity_multi("box", plan, w, t_q1, t_q2, [(score, dev(gs), codes)], params, m=m, v=v,
                                              adam=opt, grad_rows=extra)
        else:
            merged = torch.empty((plan.n_uniq, dim), device="cuda")
            fused.score_backward_entity_multi("box", plan, w, t_q1, t_q2, [(score, dev(gs), codes)], params,
                                              merged=merged, grad_rows=extra)
            fused.rows_backward(uniq_plan, merged, table=w, m=m, v=v, adam=opt)
        out[route] = (w, m, v)
    for name, a, c in zip("wmv", out["fused"], out["rows"]):
        if a is not None:
            assert torch.equal(a, c), f"{kind}: {name} differs between the fused pass and the materialised route"


def test_gradient_rows_at_a_size_that_forks():
    """4096 box queries x 300 negatives + 4096 looked-up rows, Adam: the step is large enough for the pair-ordered
    kernel (ids that occur once among the scored pairs) beside the entity pass on the second stream.  An id that is
    scored once AND looked up is no one-pair segment and must get both parts.  Against the materialised route
    (merged rows of the same call -> smx_rows_backward), bit for bit."""
    from smore_amd import fused
    n, b, k, dim, lr = 4_000_000, 4096, 300, 200, 1e-3
    g = torch.Generator(device="cuda").manual_seed(5)
    table = torch.empty((n, dim), device="cuda").uniform_(-0.07, 0.07, generator=g)
    q1 = torch.empty((b, dim), device="cuda").uniform_(-0.07, 0.07, generator=g)
    q2 = torch.empty((b, dim), device="cuda").uniform_(-0.07, 0.07, generator=g).abs_()
    idx = torch.randint(0, n, (b, k), device="cuda", generator=g)
    gs = torch.randn((b, k), device="cuda", generator=g)
    looked_up = torch.cat([idx[:, 0], torch.randint(0, n, (b // 2,), device="cuda", generator=g),
                           torch.full((300,), int(idx[0, 1]), device="cuda")])
    extra = torch.randn((looked_up.numel(), dim), device="cuda", generator=g)
    params = fused.score_params(24.0, 0.02)
    flat = torch.cat([idx.reshape(-1), looked_up])
    plan = fused.build_plan(flat, n)
    counts = torch.bincount(flat, minlength=n)
    assert int(((counts == 1)[idx.reshape(-1)]).sum().item()) > 30_000, "the case must have one-pair ids among the scored pairs"
    assert int((counts[idx[:, 0]] == 2).sum().item()) > 1000, "and ids scored once that are also looked up"
    uniq_plan = fused.build_plan(plan.uniq, n)
    out = {}
    for route in ("fused", "rows"):
        w, m, v = table.clone(), torch.zeros_like(table), torch.zeros_like(table)
        codes = fused.new_codes("box", w, idx, q1)
        score = fused.score_forward("box", w, idx, q1, q2, params, codes=codes)
        opt = fused.adam_params(lr, 2)
        if route == "fused":
            fused.score_backward_entity_multi("box", plan, w, q1, q2, [(score, gs, codes)], params, m=m, v=v, adam=opt,
                                              grad_rows=extra)
        else:
            merged = torch.empty((plan.n_uniq, dim), device="cuda")
            fused.score_backward_entity_multi("box", plan, w, q1, q2, [(score, gs, codes)], params, merged=merged,
                                              grad_rows=extra)
            fused.rows_backward(uniq_plan, merged, table=w, m=m, v=v, adam=opt)
        out[route] = (w, m, v)
    for name, a, c in zip("wmv", out["fused"], out["rows"]):
        assert torch.equal(a, c), f"{name} differs between the forking fused pass and the materialised route"
    touched = torch.zeros(n, dtype=torch.bool, device="cuda")
    touched[plan.uniq] = True
    assert torch.equal(out["fused"][0][~touched], table[~touched])
