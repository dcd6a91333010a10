"""Committed golden fixtures (tests/golden/*.npz): the oracle must reproduce them on the CPU,
the HIP path on the GPU."""
import glob
import os

import numpy as np
import pytest

from oracle import oracle as orc
from tests.util import REL_F32, assert_close, record_headroom

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "step_*.npz")))  # one per score model


def _load(path):
    d = dict(np.load(path, allow_pickle=False))
    model = os.path.basename(path)[len("step_"):-len(".npz")]
    return model, d


def test_fixtures_exist():
    assert len(GOLDEN) == 5


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
def test_oracle_reproduces_fixture(path):
    model, d = _load(path)
    w, m, v = d["table"].copy(), np.zeros_like(d["table"]), np.zeros_like(d["table"])
    q1 = d["q1"][:, None]
    q2 = d["q2"][:, None] if "q2" in d else None
    first = orc.train_step(model, w, m, v, d["idx"], q1, q2, d["gs"], float(d["gamma"]), float(d["cen"]),
                           float(d["lr"]), 1)
    orc.train_step(model, w, m, v, d["idx"], q1, q2, d["gs"], float(d["gamma"]), float(d["cen"]), float(d["lr"]), 2)
    for key in ("uniq", "inverse", "order", "seg_start"):
        assert np.array_equal(first[key], d[key]), key
    assert np.allclose(first["score"], d["score"], rtol=1e-12, atol=1e-12)
    assert np.allclose(first["merged"], d["merged"], rtol=1e-11, atol=1e-13)
    assert np.allclose(w, d["w_after"], rtol=1e-11, atol=1e-13)
    assert np.allclose(m, d["m_after"], rtol=1e-11, atol=1e-13)
    assert np.allclose(v, d["v_after"], rtol=1e-11, atol=1e-15)


@pytest.mark.gpu
@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
def test_hip_path_reproduces_fixture(path):
    import torch
    from smore_amd import fused
    model, d = _load(path)
    dev = lambda a: torch.tensor(a, dtype=torch.float32, device="cuda")
    table, q1, gs = dev(d["table"]), dev(d["q1"]), dev(d["gs"])
    q2 = dev(d["q2"]) if "q2" in d else None
    idx = torch.tensor(d["idx"], device="cuda")
    params = fused.score_params(float(d["gamma"]), float(d["cen"]))
    plan = fused.build_plan(idx, table.shape[0], want_inverse=True)
    u = plan.n_uniq
    assert np.array_equal(plan.uniq.cpu().numpy(), d["uniq"])
    assert np.array_equal(plan.inverse.cpu().numpy(), d["inverse"])
    assert np.array_equal(plan.order.cpu().numpy(), d["order"])
    assert np.array_equal(plan.seg_start[: u + 1].cpu().numpy(), d["seg_start"])
    score = fused.score_forward(model, table, idx, q1, q2, params)
    assert_close(score.cpu().numpy(), d["score"], REL_F32, "score", rms_floor=False)
    gq1, gq2 = fused.score_backward_query(model, table, idx, q1, q2, score, gs, params)
    assert_close(gq1.cpu().numpy(), d["gq1"], REL_F32, "gq1")
    if q2 is not None:
        assert_close(gq2.cpu().numpy(), d["gq2"], REL_F32, "gq2")
    merged = torch.empty((u, table.shape[1]), device="cuda")
    fused.score_backward_entity(model, plan, table, q1, q2, score, gs, params, merged=merged)
    assert_close(merged.cpu().numpy(), d["merged"], REL_F32, "merged")
    m, v = torch.zeros_like(table), torch.zeros_like(table)
    for step in (1, 2):
        score = fused.score_forward(model, table, idx, q1, q2, params)
        fused.score_backward_entity(model, plan, table, q1, q2, score, gs, params, m=m, v=v,
                                    adam=fused.adam_params(float(d["lr"]), step))
    assert_close(m.cpu().numpy(), d["m_after"], 5 * REL_F32, "m after two steps")
    err = np.abs(table.cpu().numpy() - d["w_after"])
    share = (err > 1e-5 * np.maximum(np.abs(d["w_after"]), 0.04)).mean()
    record_headroom("w after two steps: share of elements outside 1e-5 / 1e-3, worst error / (0.01 lr)", share / 1e-3,
                    err.max() / (0.01 * float(d["lr"])))
    assert err.max() < 0.01 * float(d["lr"]) and share < 1e-3      # seen: no element outside, worst error 2e-4 lr


@pytest.mark.gpu
def test_timed_path_reproduces_the_box_fixture():
    """Forward that saves sign codes + one-call backward (what bench.py times) on the box fixture."""
    import torch
    from smore_amd import fused
    _, d = _load(os.path.join(os.path.dirname(__file__), "golden", "step_box.npz"))
    dev = lambda a: torch.tensor(a, dtype=torch.float32, device="cuda")
    table, q1, q2, gs = dev(d["table"]), dev(d["q1"]), dev(d["q2"]), dev(d["gs"])
    idx = torch.tensor(d["idx"], device="cuda")
    params = fused.score_params(float(d["gamma"]), float(d["cen"]))
    plan = fused.build_plan(idx, table.shape[0])
    codes = fused.new_codes("box", table, idx, q1)
    score = fused.score_forward("box", table, idx, q1, q2, params, codes=codes)
    assert_close(score.cpu().numpy(), d["score"], REL_F32, "score", rms_floor=False)
    merged = torch.empty((plan.n_uniq, table.shape[1]), device="cuda")
    gq1, gq2 = fused.score_backward_fused("box", plan, table, idx, q1, q2, score, gs, params, merged=merged, codes=codes)
    assert_close(gq1.cpu().numpy(), d["gq1"], REL_F32, "gq1")
    assert_close(gq2.cpu().numpy(), d["gq2"], REL_F32, "gq2")
    assert_close(merged.cpu().numpy(), d["merged"], REL_F32, "merged")
    m, v = torch.zeros_like(table), torch.zeros_like(table)
    for step in (1, 2):
        score = fused.score_forward("box", table, idx, q1, q2, params, codes=codes)
        fused.score_backward_fused("box", plan, table, idx, q1, q2, score, gs, params, m=m, v=v,
                                   adam=fused.adam_params(float(d["lr"]), step), codes=codes)
    assert_close(m.cpu().numpy(), d["m_after"], 5 * REL_F32, "m after two steps")
    err = np.abs(table.cpu().numpy() - d["w_after"])
    share = (err > 1e-5 * np.maximum(np.abs(d["w_after"]), 0.04)).mean()
    record_headroom("w after two steps: share of elements outside 1e-5 / 1e-3, worst error / (0.01 lr)", share / 1e-3,
                    err.max() / (0.01 * float(d["lr"])))
    assert err.max() < 0.01 * float(d["lr"]) and share < 1e-3      # seen: no element outside, worst error 2e-4 lr


def _golden(name):
    return dict(np.load(os.path.join(os.path.dirname(__file__), "golden", name), allow_pickle=False))


def test_oracle_reproduces_loss_and_ranking_fixtures():
    d = _golden("loss.npz")
    for name, (m, w, t) in dict(plain=(None, None, 0.0), full=(d["mask"], d["weight"], float(d["temperature"]))).items():
        pl, nl, gp, gn = orc.sample_loss(d["pos"], d["neg"], m, w, t, float(d["scale"]))
        assert abs(pl - float(d[f"{name}_pos_loss"])) < 1e-13 and abs(nl - float(d[f"{name}_neg_loss"])) < 1e-13
        assert np.allclose(gp, d[f"{name}_gpos"], rtol=1e-12, atol=0) and np.allclose(gn, d[f"{name}_gneg"], rtol=1e-12, atol=0)
    r = _golden("ranking.npz")
    for i in range(r["q1"].shape[0]):
        h, e = orc.filtered_ranks(r["scores"][i], r["easy"][i].tolist(), r["hard"][i].tolist())
        assert np.array_equal(h, r["hard_ranks"][i]) and np.array_equal(e, r["easy_ranks"][i])
    c = _golden("candidates.npz")
    for i in range(c["q1"].shape[0]):
        rows = c["table"][np.where(c["neg"][i] == -1, 0, c["neg"][i])]
        logit = orc.score_forward("l1", rows[None], c["q1"][i][None, None], None, float(c["gamma"]), 0.0)[0].astype(np.float32)
        biased, ranking, filt = orc.candidate_ranks(logit, c["neg"][i], int(c["n_hard"][i]))
        assert np.array_equal(biased, c["logit"][i]) and np.array_equal(ranking, c["ranking"][i])
        assert np.array_equal(filt, c["hard_ranks"][i][: filt.size])


@pytest.mark.gpu
def test_hip_path_reproduces_loss_and_ranking_fixtures():
    import torch
    from smore_amd import fused
    from smore_amd.evaluation import filtered_ranks
    from smore_amd.training import sample_loss
    dev = lambda a: torch.tensor(a, dtype=torch.float32, device="cuda")
    d = _golden("loss.npz")
    for name, (m, w, t) in dict(plain=(None, None, 0.0), full=(d["mask"], d["weight"], float(d["temperature"]))).items():
        tp, tn = dev(d["pos"]).requires_grad_(), dev(d["neg"]).requires_grad_()
        loss, pl, nl = sample_loss(tp, tn, None if m is None else dev(m), None if w is None else dev(w), t, world_size=2)
        loss.backward()
        assert abs(pl.item() - float(d[f"{name}_pos_loss"])) <= REL_F32 * abs(float(d[f"{name}_pos_loss"]))
        assert abs(nl.item() - float(d[f"{name}_neg_loss"])) <= REL_F32 * abs(float(d[f"{name}_neg_loss"]))
        assert_close(tp.grad.cpu().numpy(), d[f"{name}_gpos"], REL_F32, "gpos")
        assert_close(tn.grad.cpu().numpy(), d[f"{name}_gneg"], REL_F32, "gneg")
    r = _golden("ranking.npz")
    got = filtered_ranks("l1", dev(r["table"]), dev(r["q1"]), None, fused.score_params(float(r["gamma"])),
                         [x.tolist() for x in r["easy"]], [x.tolist() for x in r["hard"]])
    for i, (h, e) in enumerate(got):
        assert h.cpu().numpy().tolist() == r["hard_ranks"][i].tolist()
        assert e.cpu().numpy().tolist() == r["easy_ranks"][i].tolist()
    c = _golden("candidates.npz")
    from smore_amd.evaluation import candidate_ranks
    logit, ranking, hard = candidate_ranks("l1", dev(c["table"]), dev(c["q1"]), None, fused.score_params(float(c["gamma"])),
                                           torch.tensor(c["neg"], device="cuda"), c["n_hard"])
    assert np.array_equal(logit.cpu().numpy(), c["logit"]) and np.array_equal(ranking.cpu().numpy(), c["ranking"])
    assert np.array_equal(hard.cpu().numpy(), c["hard_ranks"])
