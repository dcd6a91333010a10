"""Union queries through the C ABI: the maximum over the branches inside the scorer, the winner array that routes
both backward passes, the plan over B*K pairs (not B*U*K); against the float64 oracle's restatement of
custom_cal_logit (box.py:157-164 and siblings) and torch.max's gradient routing."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests.test_fused_gpu import GAMMA, dev, make_problem
from tests.util import REL_F32, assert_close, oracle_union_grads, oracle_union_logits, seed

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("model,n,b,u,k,dim", [("box", 300, 6, 2, 70, 48), ("l1", 100, 5, 3, 33, 200), ("rotate", 80, 4, 2, 20, 500),
                                              ("beta_kl", 90, 3, 2, 24, 64), ("l2", 120, 7, 4, 65, 36),
                                              ("distmult", 60, 2, 2, 9, 30),
                                              ("box", 200, 5, 1, 40, 48)])    # one branch: a plain query through the union calls
def test_union_forward_and_both_backwards_match_oracle(model, n, b, u, k, dim):
    from smore_amd import fused
    rng = np.random.default_rng(seed("union", model, n, b, u, k, dim))
    table, q1, q2, idx, gs = make_problem(model, n, b * u, k, dim, rng)
    idx, gs = idx[:b], gs[:b]
    idx[0, 1] = idx[0, 0]                                   # a repeated entity inside one query
    q1[1] = q1[0]                                           # two equal branches of query 0: the first one wins every pair
    if q2 is not None:
        q2[1] = q2[0]
    cen = 0.02
    params = fused.score_params(GAMMA[model], cen)
    t_table, t_q1, t_q2, t_gs = dev(table), dev(q1), dev(q2), dev(gs)
    t_idx = torch.tensor(idx, device="cuda")
    err = fused.new_error_flag("cuda")
    score, winner = fused.score_forward_union(model, t_table, t_idx, t_q1, t_q2, params, u, err)
    assert err.item() == 0 and score.shape == (b, k) and winner.dtype == torch.uint8

    qs = [q1.reshape(b, u, 1, dim)] + ([] if q2 is None else [q2.reshape(b, u, 1, dim)])
    logit, rows = oracle_union_logits(model, table, idx, qs, GAMMA[model], cen)        # [B, U, K]
    assert_close(score.cpu().numpy(), logit.max(axis=1), REL_F32, f"{model} union score",
                 rms_floor=model in ("beta_kl", "complex", "distmult"))
    # the winner is the first maximal branch of the device's own branch logits (the same kernel, one branch at a time)
    ids_rep = torch.tensor(np.repeat(idx, u, axis=0), device="cuda")
    branch = fused.score_forward(model, t_table, ids_rep, t_q1, t_q2, params, err).view(b, u, k)
    v, i = torch.max(branch, dim=1)
    assert torch.equal(score, v) and torch.equal(winner.long(), i)
    assert not (winner[0] == 1).any(), "equal branches 0 and 1: the first one takes the pair"
    win = winner.cpu().numpy().astype(np.int64)

    # both backward passes against the oracle routed by the device's winners
    g_rows = np.zeros((b, k, rows.shape[-1]))
    g_qs = [np.zeros_like(q) for q in qs]
    for j in range(u):
        gj = np.where(win == j, gs, 0.0)
        gr, g1, g2 = orc.score_backward(model, gj, rows, qs[0][:, j], qs[1][:, j] if len(qs) > 1 else None, cen)
        if model == "l2":                                   # a losing branch contributes exact zeros, not 0 * inf
            gr, g1 = np.where((win == j)[:, :, None], gr, 0.0), g1
        g_rows += gr
        g_qs[0][:, j] = g1
        if len(qs) > 1:
            g_qs[1][:, j] = g2
    gq1, gq2 = fused.score_backward_query_union(model, t_table, t_idx, t_q1, t_q2, score, t_gs, winner, params, u)
    q_abs = None if model == "beta_kl" else np.abs(gs).sum(axis=1)[:, None, None] * np.ones((1, u, dim))
    assert_close(gq1.view(b, u, dim).cpu().numpy(), g_qs[0][:, :, 0], REL_F32, f"{model} union gq1", sum_abs=q_abs)
    if q2 is not None:
        assert_close(gq2.view(b, u, dim).cpu().numpy(), g_qs[1][:, :, 0], REL_F32, f"{model} union gq2", sum_abs=q_abs)
    losers = torch.tensor(~np.any(win[:, None, :] == np.arange(u)[None, :, None], axis=2), device="cuda")
    assert not gq1.view(b, u, dim)[losers].any(), "a branch that won no pair gets an exactly zero gradient"

    plan = fused.build_plan(t_idx, n, err_flag=err)                         # B * K pairs
    uniq, inverse, _, _ = orc.merge_indices(idx)
    assert plan.n_pairs == b * k and plan.n_uniq == uniq.size
    merged = torch.full((uniq.size, table.shape[1]), float("nan"), device="cuda")
    fused.score_backward_entity_multi(model, plan, t_table, t_q1, t_q2, [(score, t_gs, None, winner)], params,
                                      merged=merged, branches=u)
    o_merged = orc.merge_grads(g_rows.reshape(b * k, -1), inverse, uniq.size)
    o_abs = orc.merge_grads(np.abs(g_rows).reshape(b * k, -1), inverse, uniq.size)
    assert_close(merged.cpu().numpy(), o_merged, REL_F32, f"{model} union merged rows", sum_abs=o_abs)
    # ... and with Adam, two streams (positives [B,1] beside the negatives) behind one plan
    pos = rng.integers(0, n, (b, 1)).astype(np.int64)
    gp = rng.standard_normal((b, 1)).astype(np.float32).astype(np.float64)
    t_pos = torch.tensor(pos, device="cuda")
    sp, wp = fused.score_forward_union(model, t_table, t_pos, t_q1, t_q2, params, u, err)
    lp, rows_p = oracle_union_logits(model, table, pos, qs, GAMMA[model], cen)
    grp, _ = oracle_union_grads(model, table, pos, qs, rows_p, lp, gp, cen)
    both = fused.build_plan(torch.cat([t_pos.reshape(-1), t_idx.reshape(-1)]), n, err_flag=err)
    uq, inv, _, _ = orc.merge_indices(np.concatenate([pos.reshape(-1), idx.reshape(-1)]))
    merged2 = torch.full((uq.size, table.shape[1]), float("nan"), device="cuda")
    fused.score_backward_entity_multi(model, both, t_table, t_q1, t_q2, [(sp, dev(gp), None, wp), (score, t_gs, None, winner)],
                                      params, merged=merged2, branches=u)
    all_rows = np.concatenate([grp, g_rows.reshape(b * k, -1)])
    assert np.array_equal(wp.cpu().numpy().astype(np.int64), np.argmax(lp, axis=1)) or model in ("beta_kl",)
    assert_close(merged2.cpu().numpy(), orc.merge_grads(all_rows, inv, uq.size), REL_F32, f"{model} union, two streams",
                 sum_abs=orc.merge_grads(np.abs(all_rows), inv, uq.size))
    assert err.item() == 0
