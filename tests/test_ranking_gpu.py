"""All-entity filtered ranking (smx_rank_answer_keys + smx_rank_scan) against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests.test_fused_gpu import GAMMA, dev, make_problem
from tests.util import REL_F32, assert_close

pytestmark = pytest.mark.gpu


def _alias(model):
    """complex_norm / distmult_norm: the model with the halves of every entity row / the whole row at unit length
    (complex.py:142-146, distmult.py:129-130)"""
    return (model[:-5], True) if model.endswith("_norm") else (model, False)


def _scores64(model, table, q1, q2, cen, norm=False):
    """float64 logits of every entity for every query, [B, N]"""
    b = q1.shape[0]
    rows = np.broadcast_to(table[None], (b,) + table.shape)
    return orc.score_forward(model, rows, q1[:, None], None if q2 is None else q2[:, None], GAMMA[model], cen, norm=norm)


def test_integer_valued_l1_ranks_are_exact_ties_included():
    """Small integer coordinates: every fp32 sum is exact, scores tie in large numbers, and the ranks
    must be exactly those of the stable descending order."""
    from smore_amd import fused
    from smore_amd.evaluation import filtered_ranks
    rng = np.random.default_rng(0)
    n, d, b = 5000, 16, 7   # passes of four, two and one queries
    table = rng.integers(-3, 4, (n, d)).astype(np.float64)
    q1 = rng.integers(-3, 4, (b, d)).astype(np.float64)
    easy = [[3, 77, 4000], [], [11], [5], [], [1, 2, 3], [4998]]
    hard = [[9, 2500, 4999, 0], [123], list(range(100, 180)),       # 80 answers: two compare chunks
            list(range(200, 270)), [42], [4999], [0, 17]]
    params = fused.score_params(GAMMA["l1"], 0.0)
    got = filtered_ranks("l1", dev(table), dev(q1), None, params, easy, hard)
    scores = _scores64("l1", table, q1, None, 0.0)
    assert len(np.unique(scores[0])) < n // 10                       # plenty of exact ties
    for i in range(b):
        want_h, want_e = orc.filtered_ranks(scores[i], easy[i], hard[i])
        assert got[i][0].cpu().numpy().tolist() == want_h.tolist()
        assert got[i][1].cpu().numpy().tolist() == want_e.tolist()


@pytest.mark.parametrize("model,dim", [("box", 200), ("l2", 64), ("rotate", 100), ("beta_kl", 40), ("box", 30), ("complex", 48),
                                       ("distmult", 64), ("beta_kl", 30), ("complex_norm", 48), ("complex_norm", 200),
                                       ("distmult_norm", 64), ("distmult_norm", 30)])
def test_ranks_lie_in_the_interval_fp32_allows(model, dim):
    """Random floats: an entity whose logit is within fp32 error of an answer's may fall on either side;
    every rank must lie between the counts with the tolerance subtracted and added."""
    from smore_amd import fused
    from smore_amd.evaluation import filtered_ranks, ranking_metrics
    rng = np.random.default_rng(dim)
    n, b = 20000, 5
    model, norm = _alias(model)
    table, q1, q2, _, _ = make_problem(model, n, b, 1, dim, rng)
    easy = [rng.choice(n, size=s, replace=False).tolist() for s in (0, 3, 10, 1, 64)]
    hard = []
    for e, s in zip(easy, (1, 5, 70, 0, 130)):
        pool = np.setdiff1d(np.arange(n), np.array(e, dtype=np.int64))
        hard.append(rng.choice(pool, size=s, replace=False).tolist())
    params = fused.score_params(GAMMA[model], 0.02, norm=norm)
    got = filtered_ranks(model, dev(table), dev(q1), dev(q2), params, easy, hard)
    scores = _scores64(model, table, q1, q2, 0.02, norm)
    for i in range(b):
        is_ans = np.zeros(n, bool)
        is_ans[easy[i] + hard[i]] = True
        tol = 2e-5 * max(1.0, np.abs(scores[i]).max())
        others = np.sort(scores[i][~is_ans])
        for ids, ranks in ((hard[i], got[i][0]), (easy[i], got[i][1])):
            r = ranks.cpu().numpy()
            assert r.shape == (len(ids),)
            for a, ra in zip(ids, r):
                lo = 1 + (others.size - np.searchsorted(others, scores[i][a] + tol, side="right"))
                hi = 1 + (others.size - np.searchsorted(others, scores[i][a] - tol, side="left"))
                assert lo <= ra <= hi, (model, i, a, ra, lo, hi)
        m = ranking_metrics(got[i][0])
        if hard[i]:
            rr = got[i][0].cpu().numpy().astype(np.float64)
            # (the metrics are fp32 means, as in the reference: train_process.py:150-154)
            assert abs(m["MRR"] - (1 / rr).mean()) < 1e-6 and abs(m["HITS10"] - (rr <= 10).mean()) < 1e-6
        else:
            assert m == dict(MRR=0.0, HITS1=0.0, HITS3=0.0, HITS10=0.0, HITS1max=0.0)


def test_planted_best_entity_and_duplicates_of_it():
    """An entity equal to the box centre inside the box has distance 0: it ranks first; copies of it at
    higher ids rank right behind it, in id order."""
    from smore_amd import fused
    from smore_amd.evaluation import filtered_ranks
    rng = np.random.default_rng(4)
    n, d = 3000, 64
    table, q1, q2, _, _ = make_problem("box", n, 1, 1, d, rng)
    for i in (10, 500, 2999):
        table[i] = q1[0]
    params = fused.score_params(24.0, 0.02)
    got = filtered_ranks("box", dev(table), dev(q1), dev(q2), params, [[]], [[500]])
    assert got[0][0].tolist() == [2]                                # entity 10 ties and has the lower id
    got = filtered_ranks("box", dev(table), dev(q1), dev(q2), params, [[10]], [[2999, 500]])
    assert got[0][0].tolist() == [1, 1] and got[0][1].tolist() == [1]  # filtered: answers do not count


@pytest.mark.parametrize("n", [1, 2, 3, 5, 9])
def test_tables_shorter_than_one_request_group(n):
    """Fewer rows than a wavefront requests at a time: the repeated last rows must not be counted."""
    from smore_amd import fused
    from smore_amd.evaluation import filtered_ranks
    rng = np.random.default_rng(n)
    d = 12
    table = rng.integers(-3, 4, (n, d)).astype(np.float64)
    q1 = rng.integers(-3, 4, (2, d)).astype(np.float64)
    hard = [[n - 1], [0]]
    got = filtered_ranks("l1", dev(table), dev(q1), None, fused.score_params(GAMMA["l1"], 0.0), [[], []], hard)
    scores = _scores64("l1", table, q1, None, 0.0)
    for i in range(2):
        want_h, _ = orc.filtered_ranks(scores[i], [], hard[i])
        assert got[i][0].cpu().numpy().tolist() == want_h.tolist()


def test_ranking_argument_errors():
    from smore_amd import _lib, fused
    from smore_amd.evaluation import filtered_ranks
    t = torch.zeros(50, 8, device="cuda")
    q = torch.zeros(1, 8, device="cuda")
    p = fused.score_params(1.0)
    with pytest.raises(IndexError):
        filtered_ranks("l1", t, q, None, p, [[]], [[50]])
    with pytest.raises(_lib.SmxError):
        filtered_ranks("l1", t, q, None, p, [[3]], [[3]])
    with pytest.raises(_lib.SmxError):
        filtered_ranks("l1", t, q, None, p, [[]], [[1], [2]])
    with pytest.raises(_lib.SmxError, match="answers per query"):
        filtered_ranks("l1", torch.zeros(4000, 8, device="cuda"), q, None, p, [[]], [list(range(2049))])


@pytest.mark.parametrize("model,dim", [("box", 64), ("rotate", 40), ("beta_kl", 36), ("l2", 200), ("distmult", 30),
                                       ("complex_norm", 52), ("distmult_norm", 44)])
def test_sampled_candidates_follow_the_reference_recipe(model, dim):
    """The sampled-negatives branch of test_step_mp (train_process.py:118-128, 141-147): -1 padding scored as entity
    0 with the -1e6 bias, ranking among the candidates, filtered ranks of the leading hard answers.  The logits
    against the float64 oracle; ranking and filtered ranks exactly the oracle's recipe applied to the device's own
    fp32 logits (two logits within rounding of each other may legitimately swap between precisions)."""
    from smore_amd import fused
    from smore_amd.evaluation import candidate_ranks
    from tests.test_fused_gpu import GAMMA, make_problem
    rng = np.random.default_rng(dim)
    n, b, c = 500, 5, 333
    model, norm = _alias(model)
    table, q1, q2, _, _ = make_problem(model, n, b, 1, dim, rng)
    neg = rng.integers(0, n, (b, c)).astype(np.int64)
    neg[0, 100:] = -1
    neg[1, 0] = -1
    neg[2, 7] = neg[2, 3]
    n_hard = np.array([4, 1, 9, 0, 333], dtype=np.int32)
    dev = lambda a: None if a is None else torch.tensor(a, dtype=torch.float32, device="cuda")
    params = fused.score_params(GAMMA[model], 0.02, norm=norm)
    err = fused.new_error_flag("cuda")
    logit, ranking, hard = candidate_ranks(model, dev(table), dev(q1), dev(q2), params, torch.tensor(neg, device="cuda"),
                                           n_hard, err)
    assert err.item() == 0
    rows = table[np.where(neg == -1, 0, neg)]
    want = orc.score_forward(model, rows, q1[:, None], None if q2 is None else q2[:, None], GAMMA[model], 0.02, norm=norm)
    want = want + np.where(neg == -1, -1e6, 0.0)
    assert_close(logit.cpu().numpy(), want, REL_F32, f"{model} candidate logits")
    got_logit = logit.cpu().numpy()
    for i in range(b):
        _, rk, filt = orc.candidate_ranks(np.where(neg[i] == -1, got_logit[i] + np.float32(1e6), got_logit[i]), neg[i],
                                          int(n_hard[i]))
        # (the bias is already in the device's logits; candidate_ranks adds it again to the un-biased copy: for a
        # padded slot fl(fl(x - 1e6) + 1e6) - 1e6 keeps the order among padded slots, which hold one value anyway)
        assert np.array_equal(ranking[i].cpu().numpy(), rk), f"{model} ranking of query {i}"
        assert np.array_equal(hard[i, : filt.size].cpu().numpy(), filt) and not hard[i, filt.size:].any()
    bad = torch.tensor(neg, device="cuda")
    bad[3, 5] = n + 4
    candidate_ranks(model, dev(table), dev(q1), dev(q2), params, bad, n_hard, err)
    assert err.item() == 1


def _union_scores64(model, table, q1, q2, cen, u, norm=False):
    """float64 logits of union queries: q1 / q2 [B, U, dim], the maximum over the branches (box.py:163), [B, N]"""
    b = q1.shape[0]
    per = [_scores64(model, table, q1[:, j], None if q2 is None else q2[:, j], cen, norm) for j in range(u)]
    return np.max(np.stack(per, axis=1), axis=1).reshape(b, -1)


@pytest.mark.parametrize("u", [2, 3, 4])
def test_union_queries_rank_exactly_by_the_maximum_over_branches(u):
    """Integer coordinates (every fp32 sum exact, many ties): the filtered ranks of a union query are those of
    max_u logit_u in the stable descending order -- not the best of the branches' own ranks."""
    from smore_amd import fused
    from smore_amd.evaluation import filtered_ranks
    rng = np.random.default_rng(u)
    n, d, b = 4000, 16, 5
    table = rng.integers(-3, 4, (n, d)).astype(np.float64)
    q1 = rng.integers(-3, 4, (b, u, d)).astype(np.float64)
    q1[1, 1] = q1[1, 0]                                   # two equal branches
    easy = [[3, 77, 3000], [], [11], [5], [1, 2]]
    hard = [[9, 2500, 3999, 0], [123], list(range(100, 180)), list(range(200, 270)), [42]]
    params = fused.score_params(GAMMA["l1"], 0.0)
    got = filtered_ranks("l1", dev(table), dev(q1), None, params, easy, hard, branches=u)
    scores = _union_scores64("l1", table, q1, None, 0.0, u)
    differs = 0
    for i in range(b):
        want_h, want_e = orc.filtered_ranks(scores[i], easy[i], hard[i])
        assert got[i][0].cpu().numpy().tolist() == want_h.tolist()
        assert got[i][1].cpu().numpy().tolist() == want_e.tolist()
        best_branch = np.min([orc.filtered_ranks(_scores64("l1", table, q1[i:i + 1, j], None, 0.0)[0], easy[i], hard[i])[0]
                              for j in range(u)], axis=0)
        differs += int((best_branch != want_h).any())
    assert differs > 0, "the case must tell the rank of the maximum from the best rank of a branch"


@pytest.mark.parametrize("model,dim,u", [("box", 200, 2), ("rotate", 100, 2), ("beta_kl", 40, 2), ("l2", 64, 3), ("distmult", 64, 4),
                                         ("box", 400, 2), ("l1", 30, 3), ("complex_norm", 48, 2), ("complex_norm", 100, 3),
                                         ("distmult_norm", 64, 4)])
def test_union_ranks_lie_in_the_interval_fp32_allows(model, dim, u):
    """Random floats, union queries: every rank between the counts with the fp32 tolerance subtracted and added;
    the answers' logits against the float64 maximum over the branches."""
    from smore_amd import fused
    from smore_amd.evaluation import filtered_ranks
    rng = np.random.default_rng(dim + u)
    n, b = 6000, 3
    model, norm = _alias(model)
    table, q1, q2, _, _ = make_problem(model, n, b * u, 1, dim, rng)
    q1 = q1.reshape(b, u, dim)
    q2 = None if q2 is None else q2.reshape(b, u, dim)
    easy = [rng.choice(n, size=s, replace=False).tolist() for s in (0, 3, 10)]
    hard = []
    for e, s in zip(easy, (1, 5, 70)):
        pool = np.setdiff1d(np.arange(n), np.array(e, dtype=np.int64))
        hard.append(rng.choice(pool, size=s, replace=False).tolist())
    params = fused.score_params(GAMMA[model], 0.02, norm=norm)
    got = filtered_ranks(model, dev(table), dev(q1), dev(q2), params, easy, hard, branches=u)
    scores = _union_scores64(model, table, q1, q2, 0.02, u, norm)
    for i in range(b):
        is_ans = np.zeros(n, bool)
        is_ans[easy[i] + hard[i]] = True
        tol = 2e-5 * max(1.0, np.abs(scores[i]).max())
        others = np.sort(scores[i][~is_ans])
        for ids, ranks in ((hard[i], got[i][0]), (easy[i], got[i][1])):
            for a, ra in zip(ids, ranks.cpu().numpy()):
                lo = 1 + (others.size - np.searchsorted(others, scores[i][a] + tol, side="right"))
                hi = 1 + (others.size - np.searchsorted(others, scores[i][a] - tol, side="left"))
                assert lo <= ra <= hi, (model, i, a, ra, lo, hi)


def test_union_of_many_branches_over_long_rows_is_refused():
    from smore_amd import _lib, fused
    from smore_amd.evaluation import filtered_ranks
    rng = np.random.default_rng(1)
    table, q1, q2, _, _ = make_problem("rotate", 50, 3, 1, 400, rng)       # rows of 800 floats: two branches at most
    params = fused.score_params(GAMMA["rotate"], 0.02)
    with pytest.raises(_lib.SmxError):
        filtered_ranks("rotate", dev(table), dev(q1.reshape(1, 3, 400)), dev(q2.reshape(1, 3, 400)), params, [[1]], [[2]],
                       branches=3)
    five = dev(rng.uniform(-0.07, 0.07, (1, 5, 400)))                       # more branches than the scan has register sets
    with pytest.raises(_lib.SmxError):
        filtered_ranks("l1", dev(table[:, :400]), five, None, fused.score_params(GAMMA["l1"], 0.0), [[1]], [[2]], branches=5)


@pytest.mark.parametrize("model,dim,u", [("box", 64, 2), ("rotate", 40, 3), ("l2", 200, 2)])
def test_sampled_candidates_of_union_queries(model, dim, u):
    """smx_rank_candidates_union: the candidates' logits are the maximum over the branches (then the -1e6 bias on the
    padding); ranking and filtered ranks are the oracle's recipe on the device's own logits."""
    from smore_amd import fused
    from smore_amd.evaluation import candidate_ranks
    rng = np.random.default_rng(dim * u)
    n, b, c = 400, 4, 150
    table, q1, q2, _, _ = make_problem(model, n, b * u, 1, dim, rng)
    q1 = q1.reshape(b, u, dim)
    q2 = None if q2 is None else q2.reshape(b, u, dim)
    neg = rng.integers(0, n, (b, c)).astype(np.int64)
    neg[0, 100:] = -1
    neg[1, 0] = -1
    n_hard = np.array([4, 1, 9, 0], dtype=np.int32)
    params = fused.score_params(GAMMA[model], 0.02)
    err = fused.new_error_flag("cuda")
    logit, ranking, hard = candidate_ranks(model, dev(table), dev(q1), dev(q2), params, torch.tensor(neg, device="cuda"),
                                           n_hard, err, branches=u)
    assert err.item() == 0
    rows = table[np.where(neg == -1, 0, neg)]
    per = [orc.score_forward(model, rows, q1[:, j, None], None if q2 is None else q2[:, j, None], GAMMA[model], 0.02)
           for j in range(u)]
    want = np.max(np.stack(per, axis=0), axis=0) + np.where(neg == -1, -1e6, 0.0)
    assert_close(logit.cpu().numpy(), want, REL_F32, f"{model} union candidate logits")
    got_logit = logit.cpu().numpy()
    for i in range(b):
        _, rk, filt = orc.candidate_ranks(np.where(neg[i] == -1, got_logit[i] + np.float32(1e6), got_logit[i]), neg[i],
                                          int(n_hard[i]))
        assert np.array_equal(ranking[i].cpu().numpy(), rk), f"{model} ranking of query {i}"
        assert np.array_equal(hard[i, : filt.size].cpu().numpy(), filt) and not hard[i, filt.size:].any()
