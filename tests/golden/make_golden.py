"""Writes the golden fixtures in this directory from the CPU oracle (float64).

The reference holds no vectors for this path (its tests print numbers), and its implementation is
CUDA-only, so the fixtures are produced by the oracle after it has been pinned against library
routines and closed forms (tests/test_oracle_pinning.py).  They freeze one tiny training step per
score model -- inputs, scores, query gradients, the integer segment plan, merged entity gradients
and the table / Adam moments after two steps -- so that a later change of the oracle or of the HIP
path that alters any result is caught against data, not against the same formula.

loss.npz and ranking.npz do the same for the sample loss (train_process.py:194-213) and for the filtered
ranks of the all-entity evaluation (train_process.py:112-160).

    python tests/golden/make_golden.py        # rewrites tests/golden/*.npz
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle as orc  # noqa: E402

GAMMA = {"l1": 12.0, "l2": 12.0, "box": 24.0, "rotate": 9.0, "beta_kl": 60.0}


def make(model, seed):
    rng = np.random.default_rng(seed)
    n, b, k, dim, lr, cen = 48, 4, 6, 8, 1e-3, 0.02
    mul = 2 if model in ("rotate", "beta_kl") else 1
    f32 = lambda x: x.astype(np.float32).astype(np.float64)
    if model == "beta_kl":
        beta = lambda *s: np.clip(1 + rng.standard_normal(s), 0.05, 1e9)
        table, q1, q2 = beta(n, dim * mul), beta(b, dim), beta(b, dim)
    else:
        table = rng.uniform(-0.07, 0.07, (n, dim * mul))
        q1 = rng.uniform(-0.07, 0.07, (b, dim))
        q2 = None if model in ("l1", "l2") else np.abs(rng.uniform(-0.07, 0.07, (b, dim)))
    table, q1 = f32(table), f32(q1)
    q2 = None if q2 is None else f32(q2)
    idx = rng.integers(0, n // 3, (b, k)).astype(np.int64)  # repeats on purpose
    gs = f32(rng.standard_normal((b, k)))
    w, m, v = table.copy(), np.zeros_like(table), np.zeros_like(table)
    o1 = q1[:, None]
    o2 = None if q2 is None else q2[:, None]
    first = orc.train_step(model, w, m, v, idx, o1, o2, gs, GAMMA[model], cen, lr, 1)
    orc.train_step(model, w, m, v, idx, o1, o2, gs, GAMMA[model], cen, lr, 2)
    out = dict(table=table, q1=q1, idx=idx, gs=gs, gamma=GAMMA[model], cen=cen, lr=lr,
               score=first["score"], gq1=first["gq1"][:, 0], uniq=first["uniq"], inverse=first["inverse"],
               order=first["order"], seg_start=first["seg_start"], merged=first["merged"],
               w_after=w, m_after=m, v_after=v)
    if q2 is not None:
        out["q2"] = q2
        out["gq2"] = first["gq2"][:, 0]
    np.savez_compressed(os.path.join(HERE, f"step_{model}.npz"), **out)


def make_loss(seed):
    rng = np.random.default_rng(seed)
    b, k = 5, 9
    f32 = lambda x: x.astype(np.float32).astype(np.float64)
    pos, neg = f32(rng.standard_normal(b) * 3), f32(rng.standard_normal((b, k)) * 3)
    mask = (rng.random((b, k)) > 0.3).astype(np.float64)
    weight = f32(rng.random(b) + 0.1)
    out = dict(pos=pos, neg=neg, mask=mask, weight=weight, temperature=0.8, scale=0.25)
    for name, (m, w, t) in dict(plain=(None, None, 0.0), full=(mask, weight, 0.8)).items():
        pl, nl, gp, gn = orc.sample_loss(pos, neg, m, w, t, 0.25)
        out.update({f"{name}_pos_loss": pl, f"{name}_neg_loss": nl, f"{name}_gpos": gp, f"{name}_gneg": gn})
    np.savez_compressed(os.path.join(HERE, "loss.npz"), **out)


def make_ranking(seed):
    """Integer-valued L1 problem: every fp32 sum is exact, so the ranks are the same in any precision."""
    rng = np.random.default_rng(seed)
    n, d, b = 600, 8, 2
    table = rng.integers(-3, 4, (n, d)).astype(np.float64)
    q1 = rng.integers(-3, 4, (b, d)).astype(np.float64)
    easy = np.array([[4, 99, 300], [17, 18, 500]], dtype=np.int64)
    hard = np.array([[7, 250, 599, 0], [1, 2, 3, 400]], dtype=np.int64)
    rows = np.broadcast_to(table[None], (b, n, d))
    scores = orc.score_forward("l1", rows, q1[:, None], None, GAMMA["l1"], 0.0)
    hr, er = zip(*(orc.filtered_ranks(scores[i], easy[i].tolist(), hard[i].tolist()) for i in range(b)))
    np.savez_compressed(os.path.join(HERE, "ranking.npz"), table=table, q1=q1, easy=easy, hard=hard, gamma=GAMMA["l1"],
                        scores=scores, hard_ranks=np.array(hr), easy_ranks=np.array(er))


def make_candidates(seed):
    """Sampled-candidate evaluation on an integer-valued L1 problem (exact in any precision): padding, ties, a hard
    answer that is not the best candidate."""
    rng = np.random.default_rng(seed)
    n, d, b, c = 200, 8, 3, 40
    table = rng.integers(-3, 4, (n, d)).astype(np.float64)
    q1 = rng.integers(-3, 4, (b, d)).astype(np.float64)
    neg = rng.integers(0, n, (b, c)).astype(np.int64)
    neg[0, 30:] = -1
    neg[1, [5, 6]] = neg[1, 0]          # the same entity three times: equal logits
    neg[2, 0] = -1                      # the answer is not among the candidates (train_process.py:137)
    n_hard = np.array([3, 2, 1], dtype=np.int32)
    rows = table[np.where(neg == -1, 0, neg)]
    logit = orc.score_forward("l1", rows, q1[:, None], None, GAMMA["l1"], 0.0).astype(np.float32)
    out = [orc.candidate_ranks(logit[i], neg[i], int(n_hard[i])) for i in range(b)]
    hard = np.zeros((b, 3), dtype=np.int64)
    for i, (_, _, f) in enumerate(out):
        hard[i, : f.size] = f
    np.savez_compressed(os.path.join(HERE, "candidates.npz"), table=table, q1=q1, neg=neg, n_hard=n_hard, gamma=GAMMA["l1"],
                        logit=np.stack([o[0] for o in out]), ranking=np.stack([o[1] for o in out]), hard_ranks=hard)


if __name__ == "__main__":
    for i, model in enumerate(GAMMA):
        make(model, 100 + i)
    make_loss(200)
    make_ranking(300)
    make_candidates(400)
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
