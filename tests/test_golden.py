"""Committed golden fixtures (tests/golden/step_*.npz): the oracle must reproduce them on the CPU,
the HIP path on the GPU."""
import glob
import os

import numpy as np
import pytest

from oracle import oracle as orc
from tests.util import REL_F32, assert_close

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "step_*.npz")))


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
    assert_close(score.cpu().numpy(), d["score"], REL_F32, "score")
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
    assert err.max() < 2 * float(d["lr"]) and (err > 1e-5 * np.maximum(np.abs(d["w_after"]), 0.04)).mean() < 0.01
