"""Unchanged model code on the fused path.

The classes below are a few-line restatement, written for this test, of how SMORE's models reach the scoring
path: the lookup / view / regularizer / cal_logit sequence of KGReasoning.forward (kg_reasoning.py:298-307,
340-355) and the custom_cal_logit bodies (box.py:157-164, vec.py:85-90, rotate.py:137-142, beta.py:303-308,
complex.py:140-148, distmult.py).
They call only sp_embed(ids, name), tensor methods and ext_ops -- no score_negatives -- and must get, through the
lazy lookup handle, the gather-fused scorer, with logits, query gradients and Adam state equal to the float64
oracle's."""
import types

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests.util import (REL_F32, assert_adam_weights, assert_close, oracle_adam_step, oracle_union_grads,
                        oracle_union_logits)

pytestmark = pytest.mark.gpu


class Reasoner(torch.nn.Module):
    def __init__(self, entity_embedding, gamma):
        super().__init__()
        self.entity_embedding = entity_embedding
        self.gamma = torch.nn.Parameter(torch.Tensor([gamma]), requires_grad=False)

    def entity_regularizer(self, embedding):
        return embedding

    def forward(self, positive_sample, negative_sample, query_embedding):
        all_positive = self.entity_embedding(positive_sample, "positive_entity")
        batch_size, negative_size = negative_sample.shape
        all_negative = self.entity_embedding(negative_sample.view(-1), "negative_entity")
        all_positive.job_handle.sync()
        all_positive = self.entity_regularizer(all_positive)
        positive_logits = self.cal_logit(all_positive.unsqueeze(1), None, query_embedding)
        all_negative.job_handle.sync()
        all_negative = self.entity_regularizer(all_negative.view(batch_size, negative_size, -1))
        negative_logits = self.cal_logit(all_negative, None, query_embedding)
        return positive_logits, negative_logits


class Box(Reasoner):
    cen = 0.02

    def cal_logit(self, entity_embedding, entity_feat, query_embedding):
        from smore_amd.torchext.ext_ops import box_dist_in, box_dist_out
        assert entity_feat is None
        center, offset = query_embedding
        d1 = box_dist_out(entity_embedding, center, offset)
        d2 = box_dist_in(entity_embedding, center, offset)
        logit = self.gamma - d1 - self.cen * d2
        return torch.max(logit, dim=1)[0]


class Vec(Reasoner):
    def __init__(self, entity_embedding, gamma, mode):
        super().__init__(entity_embedding, gamma)
        from smore_amd.torchext import ext_ops
        self.dist_func = getattr(ext_ops, mode + "_dist")

    def cal_logit(self, entity_embedding, entity_feat, query_embedding):
        assert entity_feat is None
        logit = self.gamma - self.dist_func(entity_embedding, query_embedding[0])
        return torch.max(logit, dim=1)[0]


class Rotate(Reasoner):
    def cal_logit(self, entity_embedding, entity_feat, query_embedding):
        from smore_amd.torchext.ext_ops import rotate_dist
        assert entity_feat is None
        re, im = query_embedding
        logit = self.gamma - rotate_dist(entity_embedding, re, im)
        return torch.max(logit, dim=1)[0]


class Beta(Reasoner):
    def entity_regularizer(self, embedding):      # Regularizer(1, 0.05, 1e9), beta.py:210, modules.py:29-36
        return torch.clamp(embedding + 1.0, 0.05, 1e9)

    def cal_logit(self, entity_embedding, entity_feat, query_embedding):
        from smore_amd.torchext.ext_ops import BetaDist, beta_kl
        assert entity_feat is None
        logit = self.gamma - beta_kl(entity_embedding, BetaDist(*query_embedding))
        return torch.max(logit, dim=1)[0]


class BetaNative(Beta):            # native_cal_logit, beta.py:293-301: torch's own Beta-Beta KL routine on the halves
    def cal_logit(self, entity_embedding, entity_feat, query_embedding):
        import torch.distributions.kl as torch_kl
        from smore_amd.torchext.ext_ops import BetaDist
        assert entity_feat is None
        alpha_embedding, beta_embedding = torch.chunk(entity_embedding.unsqueeze(1), 2, dim=-1)
        entity_dist = BetaDist(alpha_embedding, beta_embedding)
        query_dist = BetaDist(*query_embedding)
        kld = torch_kl._kl_beta_beta(entity_dist, query_dist)
        logit = self.gamma - torch.norm(kld, p=1, dim=-1)
        logit = torch.max(logit, dim=1)[0]
        return logit


class Complex(Reasoner):                           # complex.py:140-148 without its optional normalisation
    def cal_logit(self, entity_embedding, entity_feat, query_embedding):
        from smore_amd.torchext.ext_ops import complex_sim
        assert entity_feat is None
        re, im = query_embedding
        logit = complex_sim(entity_embedding, re, im)
        return torch.max(logit, dim=1)[0]


class ComplexNorm(Reasoner):       # complex.py:140-148 in its 'norm' mode (complex.py:87-89; Normalizer, modules.py:38-40)
    need_norm = True

    @staticmethod
    def embed_norm(embedding):
        return torch.nn.functional.normalize(embedding, p=2, dim=-1)

    def cal_logit(self, entity_embedding, entity_feat, query_embedding):
        from smore_amd.torchext.ext_ops import complex_sim
        assert entity_feat is None
        query_re_embedding, query_im_embedding = query_embedding
        if self.need_norm:
            entity_re_embedding, entity_im_embedding = torch.chunk(entity_embedding, 2, dim=-1)
            entity_re_embedding, entity_im_embedding = self.embed_norm(entity_re_embedding), self.embed_norm(entity_im_embedding)
            entity_embedding = torch.cat((entity_re_embedding, entity_im_embedding), dim=-1).contiguous()
        logit = complex_sim(entity_embedding, query_re_embedding, query_im_embedding)
        return torch.max(logit, dim=1)[0]


class BoxNative(Reasoner):         # native_cal_logit, box.py:147-155 (--logit_impl native, the scripts' default)
    cen = 0.02

    def cal_logit(self, entity_embedding, entity_feat, query_embedding):
        F = torch.nn.functional
        assert entity_feat is None
        query_center_embedding, query_offset_embedding = query_embedding
        delta = (entity_embedding.unsqueeze(1) - query_center_embedding).abs()
        distance_out = F.relu(delta - query_offset_embedding)
        distance_in = torch.min(delta, query_offset_embedding)
        logit = self.gamma - torch.norm(distance_out, p=1, dim=-1) - self.cen * torch.norm(distance_in, p=1, dim=-1)
        logit = torch.max(logit, dim=1)[0]
        return logit


class VecNative(Reasoner):         # native_cal_logit, vec.py:78-83
    def cal_logit(self, entity_embedding, entity_feat, query_embedding):
        assert entity_feat is None
        distance = entity_embedding.unsqueeze(1) - query_embedding[0]
        logit = self.gamma - torch.norm(distance, p=1, dim=-1)
        logit = torch.max(logit, dim=1)[0]
        return logit


class RotateNative(Reasoner):      # native_cal_logit, rotate.py:125-135
    def cal_logit(self, entity_embedding, entity_feat, query_embedding):
        assert entity_feat is None
        query_re_embedding, query_im_embedding = query_embedding
        entity_re_embedding, entity_im_embedding = torch.chunk(entity_embedding.unsqueeze(1), 2, dim=-1)
        re_distance = entity_re_embedding - query_re_embedding
        im_distance = entity_im_embedding - query_im_embedding
        distance = torch.stack([re_distance, im_distance], dim=0)
        distance = distance.norm(dim=0)
        logit = self.gamma - distance.sum(dim=-1)
        logit = torch.max(logit, dim=1)[0]
        return logit


class DistmultNative(Reasoner):    # native_cal_logit, distmult.py:126-133 (the model's only form)
    need_norm = False

    @staticmethod
    def embed_norm(embedding):     # Normalizer, modules.py:38-40
        return torch.nn.functional.normalize(embedding, p=2, dim=-1)

    def cal_logit(self, entity_embedding, entity_feat, query_embedding):
        assert entity_feat is None
        entity_embedding = entity_embedding.unsqueeze(1)
        if self.need_norm:
            entity_embedding = self.embed_norm(entity_embedding)
        logit = (query_embedding[0] * entity_embedding).sum(-1)
        logit = torch.max(logit, dim=1)[0]
        return logit


class DistmultNativeNorm(DistmultNative):      # -distmultm '(Mean,True,norm)', three of the reference's scripts
    need_norm = True


class ComplexNative(Reasoner):     # native_cal_logit, complex.py:169-177: rows of the queries' own batch
    need_norm = False
    embed_norm = staticmethod(ComplexNorm.embed_norm)

    def cal_logit(self, entity_embedding, entity_feat, query_embedding):
        assert entity_feat is None
        query_re_embedding, query_im_embedding = query_embedding
        entity_re_embedding, entity_im_embedding = torch.chunk(entity_embedding.unsqueeze(1), 2, dim=-1)
        if self.need_norm:
            entity_re_embedding, entity_im_embedding = self.embed_norm(entity_re_embedding), self.embed_norm(entity_im_embedding)
        assert entity_re_embedding.shape[0] == query_re_embedding.shape[0]
        logit = (entity_re_embedding * query_re_embedding + entity_im_embedding * query_im_embedding).sum(dim=-1)
        logit = torch.max(logit, dim=1)[0]
        return logit


class ComplexNativeNorm(ComplexNative):
    need_norm = True


class Distmult(Reasoner):
    def cal_logit(self, entity_embedding, entity_feat, query_embedding):
        from smore_amd.torchext.ext_ops import distmult_sim
        assert entity_feat is None
        logit = distmult_sim(entity_embedding, query_embedding[0])
        return torch.max(logit, dim=1)[0]


CASES = {
    # name: (class, extra ctor args, fused model, queries per branch, row / dim, gamma, cen)
    "box": (Box, (), "box", 2, 1, 24.0, 0.02),
    "l1": (Vec, ("l1",), "l1", 1, 1, 12.0, 0.0),
    "l2": (Vec, ("l2",), "l2", 1, 1, 12.0, 0.0),
    "rotate": (Rotate, (), "rotate", 2, 2, 9.0, 0.0),
    "beta": (Beta, (), "beta_kl", 2, 2, 60.0, 0.0),
    "complex": (Complex, (), "complex", 2, 2, 0.0, 0.0),
    "distmult": (Distmult, (), "distmult", 1, 1, 0.0, 0.0),
    "complex_norm": (ComplexNorm, (), "complex", 2, 2, 0.0, 0.0),
    "box_native": (BoxNative, (), "box", 2, 1, 24.0, 0.02),
    "l1_native": (VecNative, (), "l1", 1, 1, 12.0, 0.0),
    "rotate_native": (RotateNative, (), "rotate", 2, 2, 9.0, 0.0),
    "distmult_native": (DistmultNative, (), "distmult", 1, 1, 0.0, 0.0),
    "complex_native": (ComplexNative, (), "complex", 2, 2, 0.0, 0.0),
    "complex_norm_native": (ComplexNativeNorm, (), "complex", 2, 2, 0.0, 0.0),
    "distmult_norm_native": (DistmultNativeNorm, (), "distmult", 1, 1, 0.0, 0.0),
    "beta_native": (BetaNative, (), "beta_kl", 2, 2, 60.0, 0.0),
}


def _table_and_queries(name, n, d, b, u, rng):
    mul = CASES[name][4]
    n_q = CASES[name][3]
    if name.startswith("beta"):
        table = rng.standard_normal((n, 2 * d)) * 1.5           # raw values; the regularizer clamps some
        pos = lambda *s: np.clip(1 + rng.standard_normal(s), 0.05, 1e9)
        qs = [pos(b, u, 1, d) for _ in range(n_q)]
    else:
        table = rng.uniform(-0.07, 0.07, (n, mul * d))
        qs = [rng.uniform(-0.07, 0.07, (b, u, 1, d)) for _ in range(n_q)]
        if name in ("box", "box_native"):
            qs[1] = np.abs(qs[1])
    f32 = lambda a: a.astype(np.float32).astype(np.float64)
    return f32(table), [f32(q) for q in qs]


def _oracle_branch_logits(name, table, ids, qs, gamma, cen):
    return oracle_union_logits(CASES[name][2], table, ids, qs, gamma, cen, regularizer=name.startswith("beta"),
                               norm="_norm" in name)


def _oracle_grads(name, table, ids, qs, rows, logit, gout, cen):
    return oracle_union_grads(CASES[name][2], table, ids, qs, rows, logit, gout, cen, regularizer=name.startswith("beta"),
                              norm="_norm" in name)


@pytest.mark.parametrize("name", list(CASES))
@pytest.mark.parametrize("branches", [1, 2])
def test_model_code_without_score_negatives_matches_oracle(name, branches, monkeypatch):
    from smore_amd import fused
    from smore_amd.embedding.embed_optimizer import AdamEmbedOptimizer
    from smore_amd.embedding.sparse_embed import SparseEmbedding

    def no_gradient_rows(*a, **k):
        raise AssertionError("positives + negatives of one query batch must not go through materialised gradient rows")
    monkeypatch.setattr(fused, "rows_backward", no_gradient_rows)
    cls, extra, model, n_q, mul, gamma, cen = CASES[name]
    n, d, b, k, lr = 400, 32, 6, 24, 1e-3
    rng = np.random.default_rng(11 + branches)
    table, qs = _table_and_queries(name, n, d, b, branches, rng)
    emb = SparseEmbedding(n, mul * d).cuda()
    with torch.no_grad():
        emb.embedding.copy_(torch.tensor(table, dtype=torch.float32))
    opt = AdamEmbedOptimizer(types.SimpleNamespace(optim_mode="(aggr,adam,gpu,False,5)", share_optim_stats=True), emb, 0)
    net = cls(emb, gamma, *extra).cuda()
    t_qs = [torch.tensor(q, dtype=torch.float32, device="cuda", requires_grad=True) for q in qs]
    w, m, v = table.copy(), np.zeros_like(table), np.zeros_like(table)
    for step in (1, 2):
        pos = rng.integers(0, n, b)
        neg = rng.integers(0, n // 4, (b, k))                             # repeated ids: real segments
        gp = rng.standard_normal((b, 1)).astype(np.float32).astype(np.float64)
        gn = rng.standard_normal((b, k)).astype(np.float32).astype(np.float64)
        opt.zero_grad()
        for t in t_qs:
            t.grad = None
        lp, ln = net(torch.tensor(pos, device="cuda"), torch.tensor(neg, device="cuda"), t_qs)
        assert lp.shape == (b, 1) and ln.shape == (b, k)
        ((lp * torch.tensor(gp, dtype=torch.float32, device="cuda")).sum() +
         (ln * torch.tensor(gn, dtype=torch.float32, device="cuda")).sum()).backward()
        # both lookups wait for their first use (the maximum over union branches included) and share one launch
        assert len(opt.fused_list) == 1 and not opt.grad_list, "both lookups must have stayed on the fused scorer"
        opt.apply_grad(lr)

        o_lp, rows_p = _oracle_branch_logits(name, w, pos.reshape(b, 1), qs, gamma, cen)
        o_ln, rows_n = _oracle_branch_logits(name, w, neg, qs, gamma, cen)
        assert_close(lp.detach().cpu().numpy(), o_lp.max(axis=1), REL_F32, f"{name} positive logits, step {step}")
        assert_close(ln.detach().cpu().numpy(), o_ln.max(axis=1), REL_F32, f"{name} negative logits, step {step}")
        gr_p, gq_p = _oracle_grads(name, w, pos.reshape(b, 1), qs, rows_p, o_lp, gp, cen)
        gr_n, gq_n = _oracle_grads(name, w, neg, qs, rows_n, o_ln, gn, cen)
        for t, a, c in zip(t_qs, gq_p, gq_n):
            assert_close(t.grad.cpu().numpy(), a + c, REL_F32, f"{name} query gradient, step {step}")
        all_idx = np.concatenate([pos.reshape(-1), neg.reshape(-1)])
        uniq, inverse, _, _ = orc.merge_indices(all_idx)
        merged = orc.merge_grads(np.concatenate([gr_p, gr_n]), inverse, uniq.size)
        w_before = w.copy()
        orc.adam_rows(w, m, v, uniq, merged, lr, step)
        got = emb.embedding.detach().cpu().numpy().astype(np.float64)
        touched = np.zeros(n, bool)
        touched[uniq] = True
        assert np.array_equal(got[~touched], w_before[~touched]), "rows outside the step must keep their bits"
        assert_close(emb.state_sum_fo.cpu().numpy()[touched], m[touched], REL_F32, f"{name} first moment, step {step}")
        assert_close(emb.state_sum_sq.cpu().numpy()[touched], v[touched], REL_F32, f"{name} second moment, step {step}")
        assert_adam_weights(got, w, merged, uniq, lr, f"{name} weights, step {step}")
        w = got.copy()   # continue from the device's fp32 weights so that step 2 compares one step, not two
        m = emb.state_sum_fo.cpu().numpy().astype(np.float64)
        v = emb.state_sum_sq.cpu().numpy().astype(np.float64)


def test_negatives_only_step_is_the_one_record_fast_path():
    """The cfg5 call shape: negatives only.  The lazy route must leave exactly one fused record (plan + fused
    entity pass, no gradient rows) and give the bits of the explicit score_negatives call."""
    from smore_amd.embedding.embed_optimizer import AdamEmbedOptimizer
    from smore_amd.embedding.sparse_embed import SparseEmbedding
    n, d, b, k, lr = 3000, 200, 16, 64, 1e-4
    rng = np.random.default_rng(5)
    neg = torch.tensor(np.minimum(rng.zipf(1.3, (b, k)) - 1, n - 1), device="cuda")
    cn = rng.uniform(-0.07, 0.07, (b, 1, 1, d)).astype(np.float32)
    on = np.abs(rng.uniform(-0.07, 0.07, (b, 1, 1, d))).astype(np.float32)
    gn = torch.tensor(rng.standard_normal((b, k)).astype(np.float32), device="cuda")

    def run(lazy):
        torch.manual_seed(3)
        emb = SparseEmbedding(n, d).cuda()
        emb.init_params(-0.07, 0.07)
        opt = AdamEmbedOptimizer(types.SimpleNamespace(optim_mode="(aggr,adam,gpu,False,5)", share_optim_stats=True), emb, 0)
        net = Box(emb, 24.0).cuda()
        c = torch.tensor(cn, device="cuda", requires_grad=True)
        o = torch.tensor(on, device="cuda", requires_grad=True)
        for _ in range(2):
            opt.zero_grad()
            c.grad = o.grad = None
            if lazy:
                rows = emb(neg.view(-1), "negative_entity")
                rows.job_handle.sync()
                ln = net.cal_logit(net.entity_regularizer(rows.view(b, k, -1)), None, [c, o])
            else:
                ln = opt.score_negatives("box", neg, c, o, gamma=24.0, cen=0.02)
            (ln * gn).sum().backward()
            assert len(opt.fused_list) == 1 and not opt.grad_list
            opt.apply_grad(lr)
        return [x.detach().cpu() for x in (ln, c.grad, o.grad, emb.embedding, emb.state_sum_fo, emb.state_sum_sq)]

    for a, r in zip(run(True), run(False)):
        assert torch.equal(a, r)


def test_shared_negatives_and_other_uses_of_the_rows():
    """--share_negative: negative_sample is [1,K] (online_sampler.py:155-157), so batch_size = 1 in the model code
    and the operators broadcast the K rows over the B queries.  cal_reg (kg_reasoning.py:149-152) also wants the
    rows' values: the handle then looks them up once, and the step merges the two records."""
    from smore_amd.embedding.embed_optimizer import AdamEmbedOptimizer
    from smore_amd.embedding.sparse_embed import SparseEmbedding
    n, d, b, k, lr = 300, 16, 5, 12, 1e-3
    rng = np.random.default_rng(8)
    table = rng.uniform(-0.07, 0.07, (n, d)).astype(np.float32).astype(np.float64)
    q = rng.uniform(-0.07, 0.07, (b, 1, 1, d)).astype(np.float32).astype(np.float64)
    neg = rng.integers(0, n, (1, k))
    gn = rng.standard_normal((b, k)).astype(np.float32).astype(np.float64)
    emb = SparseEmbedding(n, d).cuda()
    with torch.no_grad():
        emb.embedding.copy_(torch.tensor(table, dtype=torch.float32))
    opt = AdamEmbedOptimizer(types.SimpleNamespace(optim_mode="(aggr,adam,gpu,False,5)", share_optim_stats=True), emb, 0)
    net = Vec(emb, 12.0, "l1").cuda()
    tq = torch.tensor(q, dtype=torch.float32, device="cuda", requires_grad=True)
    opt.zero_grad()
    t_neg = torch.tensor(neg, device="cuda")
    rows = emb(t_neg.view(-1), "negative_entity")
    ln = net.cal_logit(rows.view(1, k, -1), None, [tq])
    assert ln.shape == (b, k)
    reg = torch.norm(rows, p=3) ** 3
    ((ln * torch.tensor(gn, dtype=torch.float32, device="cuda")).sum() + 0.5 * reg).backward()
    assert len(opt.fused_list) == 1 and len(opt.grad_list) == 1
    opt.apply_grad(lr)

    ids_full = np.broadcast_to(neg, (b, k))
    o_rows = orc.gather(table, ids_full).reshape(b, k, d)
    assert_close(ln.detach().cpu().numpy(), orc.score_forward("l1", o_rows, q[:, 0], None, 12.0), REL_F32, "logits")
    g_rows, g_q, _ = orc.score_backward("l1", gn, o_rows, q[:, 0], None)
    assert_close(tq.grad.cpu().numpy()[:, 0], g_q, REL_F32, "query gradient")
    r = orc.gather(table, neg)
    g_reg = 0.5 * 3.0 * np.abs(r) * r                                       # d/dx |x|^3 = 3 |x| x
    all_idx = np.concatenate([ids_full.reshape(-1), neg.reshape(-1)])
    uniq, inverse, _, _ = orc.merge_indices(all_idx)
    merged = orc.merge_grads(np.concatenate([g_rows.reshape(b * k, d), g_reg]), inverse, uniq.size)
    w, m, v = table.copy(), np.zeros_like(table), np.zeros_like(table)
    orc.adam_rows(w, m, v, uniq, merged, lr, 1)
    assert_close(emb.state_sum_fo.cpu().numpy()[uniq], m[uniq], REL_F32, "first moment")
    assert_adam_weights(emb.embedding.detach().cpu().numpy(), w, merged, uniq, lr, "weights")


def test_complex_norm_step_with_shared_negatives_stays_fused():
    """The layout of the reference's ComplEx scripts (complex_scripts/train_*.sh: -complexm '(Mean,True,norm)' with
    --share_negative): negatives [1,K] and positives [B] through the unchanged custom_cal_logit of the 'norm' mode.
    No lookup is materialised, the K ids and the B positives meet in one plan, and logits, query gradients and the
    Adam step are the float64 oracle's."""
    from smore_amd.embedding.embed_optimizer import AdamEmbedOptimizer
    from smore_amd.embedding.sparse_embed import SparseEmbedding
    n, d, b, k, lr = 500, 48, 9, 70, 1e-3
    rng = np.random.default_rng(77)
    table, qs = _table_and_queries("complex_norm", n, d, b, 1, rng)
    emb = SparseEmbedding(n, 2 * d).cuda()
    with torch.no_grad():
        emb.embedding.copy_(torch.tensor(table, dtype=torch.float32))
    opt = AdamEmbedOptimizer(types.SimpleNamespace(optim_mode="(aggr,adam,gpu,False,5)", share_optim_stats=True), emb, 0)
    net = ComplexNorm(emb, 0.0).cuda()
    t_qs = [torch.tensor(q, dtype=torch.float32, device="cuda", requires_grad=True) for q in qs]
    pos = rng.integers(0, n, b)
    neg = rng.integers(0, n // 4, (1, k))
    neg[0, 5] = pos[2]                                   # an entity that is a positive and a shared negative at once
    gp = rng.standard_normal((b, 1)).astype(np.float32).astype(np.float64)
    gn = rng.standard_normal((b, k)).astype(np.float32).astype(np.float64)
    opt.zero_grad()
    lp, ln = net(torch.tensor(pos, device="cuda"), torch.tensor(neg, device="cuda"), t_qs)
    assert lp.shape == (b, 1) and ln.shape == (b, k)
    ((lp * torch.tensor(gp, dtype=torch.float32, device="cuda")).sum() +
     (ln * torch.tensor(gn, dtype=torch.float32, device="cuda")).sum()).backward()
    assert len(opt.fused_list) == 2 and not opt.grad_list and opt.stats["materialized_lookups"] == 0
    assert opt.stats["dense_fallbacks"] == 0
    opt.apply_grad(lr)

    neg_full = np.broadcast_to(neg, (b, k))
    o_lp, rows_p = _oracle_branch_logits("complex_norm", table, pos.reshape(b, 1), qs, 0.0, 0.0)
    o_ln, rows_n = _oracle_branch_logits("complex_norm", table, neg_full, qs, 0.0, 0.0)
    assert_close(lp.detach().cpu().numpy(), o_lp[:, 0], REL_F32, "positive logits")
    assert_close(ln.detach().cpu().numpy(), o_ln[:, 0], REL_F32, "negative logits")
    gr_p, gq_p = _oracle_grads("complex_norm", table, pos.reshape(b, 1), qs, rows_p, o_lp, gp, 0.0)
    gr_n, gq_n = _oracle_grads("complex_norm", table, neg_full, qs, rows_n, o_ln, gn, 0.0)
    for t, a, c in zip(t_qs, gq_p, gq_n):
        assert_close(t.grad.cpu().numpy(), a + c, REL_F32, "query gradient")
    all_idx = np.concatenate([pos.reshape(-1), neg_full.reshape(-1)])
    uniq, inverse, _, _ = orc.merge_indices(all_idx)
    merged = orc.merge_grads(np.concatenate([gr_p, gr_n]), inverse, uniq.size)
    w, m, v = table.copy(), np.zeros_like(table), np.zeros_like(table)
    orc.adam_rows(w, m, v, uniq, merged, lr, 1)
    assert_close(emb.state_sum_fo.cpu().numpy()[uniq], m[uniq], REL_F32, "first moment")
    assert_adam_weights(emb.embedding.detach().cpu().numpy(), w, merged, uniq, lr, "weights")


@pytest.mark.parametrize("native,custom,mul,n_q", [(BoxNative, Box, 1, 2), (VecNative, None, 1, 1), (RotateNative, Rotate, 2, 2)])
def test_native_bodies_with_shared_negatives_give_the_bits_of_the_ext_ops_form(native, custom, mul, n_q):
    """--share_negative with --logit_impl native (what 31 of the reference's 40 scripts run): the torch-operator
    body on a [1, K] handle asks the fused scorer for exactly what the ext_ops body asks -- same launches, same
    bits in logits, query gradients, table and optimizer state, and no lookup materialised."""
    from smore_amd.embedding.embed_optimizer import AdamEmbedOptimizer
    from smore_amd.embedding.sparse_embed import SparseEmbedding
    n, d, b, k, lr = 400, 40, 7, 90, 1e-3
    rng = np.random.default_rng(41)
    table = rng.uniform(-0.07, 0.07, (n, mul * d)).astype(np.float32)
    qs = [rng.uniform(-0.07, 0.07, (b, 1, 1, d)).astype(np.float32) for _ in range(n_q)]
    if native is BoxNative:
        qs[1] = np.abs(qs[1])
    pos, neg = rng.integers(0, n, b), rng.integers(0, n // 3, (1, k))
    gp = rng.standard_normal((b, 1)).astype(np.float32)
    gn = rng.standard_normal((b, k)).astype(np.float32)

    def run(cls, *extra):
        emb = SparseEmbedding(n, mul * d).cuda()
        with torch.no_grad():
            emb.embedding.copy_(torch.tensor(table))
        opt = AdamEmbedOptimizer(types.SimpleNamespace(optim_mode="(aggr,adam,gpu,False,5)", share_optim_stats=True), emb, 0)
        net = cls(emb, 12.0, *extra).cuda()
        t_qs = [torch.tensor(q, device="cuda", requires_grad=True) for q in qs]
        opt.zero_grad()
        lp, ln = net(torch.tensor(pos, device="cuda"), torch.tensor(neg, device="cuda"), t_qs)
        assert lp.shape == (b, 1) and ln.shape == (b, k)
        ((lp * torch.tensor(gp, device="cuda")).sum() + (ln * torch.tensor(gn, device="cuda")).sum()).backward()
        assert not opt.grad_list and opt.stats["materialized_lookups"] == 0 and opt.stats["dense_fallbacks"] == 0
        opt.apply_grad(lr)
        return [x.detach().cpu() for x in (lp, ln, *[t.grad for t in t_qs], emb.embedding, emb.state_sum_fo, emb.state_sum_sq)]

    got = run(native)
    want = run(custom) if custom is not None else run(Vec, "l1")
    for a, r in zip(got, want):
        assert torch.equal(a, r)


@pytest.mark.parametrize("need_norm", [False, True])
def test_complex_native_body_with_shared_negatives_takes_its_matrix_product_branch(need_norm):
    """What every ComplEx script of the reference runs: native_cal_logit (complex.py:169-187) with --share_negative.
    The positives [B] meet the queries' own batch; the shared negatives [1, K] take the model's torch.mm branch (the
    halves viewed as matrices, transposed, multiplied by the query matrices, added).  The handle follows both: no
    lookup is materialised and the step leaves the two fused records of the ext_ops form.  Against the oracle."""
    from smore_amd.embedding.embed_optimizer import AdamEmbedOptimizer
    from smore_amd.embedding.sparse_embed import SparseEmbedding
    F = torch.nn.functional
    n, d, b, k, lr = 300, 24, 6, 40, 1e-3
    rng = np.random.default_rng(91)
    name = "complex_norm" if need_norm else "complex"
    table, qs = _table_and_queries(name, n, d, b, 1, rng)
    emb = SparseEmbedding(n, 2 * d).cuda()
    with torch.no_grad():
        emb.embedding.copy_(torch.tensor(table, dtype=torch.float32))
    opt = AdamEmbedOptimizer(types.SimpleNamespace(optim_mode="(aggr,adam,gpu,False,5)", share_optim_stats=True), emb, 0)
    embed_norm = (lambda x: F.normalize(x, p=2, dim=-1)) if need_norm else (lambda x: x)

    def native_cal_logit(entity_embedding, query_embedding):            # complex.py:169-187
        query_re_embedding, query_im_embedding = query_embedding
        entity_re_embedding, entity_im_embedding = torch.chunk(entity_embedding.unsqueeze(1), 2, dim=-1)
        if need_norm:
            entity_re_embedding, entity_im_embedding = embed_norm(entity_re_embedding), embed_norm(entity_im_embedding)
        if entity_re_embedding.shape[0] == query_re_embedding.shape[0]:
            logit = (entity_re_embedding * query_re_embedding + entity_im_embedding * query_im_embedding).sum(dim=-1)
            logit = torch.max(logit, dim=1)[0]
        else:
            bsize = query_re_embedding.shape[0]
            nent = entity_re_embedding.shape[2]
            embed_dim = query_re_embedding.shape[-1]
            entity_re_embedding = entity_re_embedding.view(nent, embed_dim)
            entity_im_embedding = entity_im_embedding.view(nent, embed_dim)
            query_re_embedding = query_re_embedding.view(bsize, embed_dim)
            query_im_embedding = query_im_embedding.view(bsize, embed_dim)
            logit = torch.mm(query_re_embedding, entity_re_embedding.t()) + torch.mm(query_im_embedding, entity_im_embedding.t())
        return logit

    t_qs = [torch.tensor(q, dtype=torch.float32, device="cuda", requires_grad=True) for q in qs]
    pos, neg = rng.integers(0, n, b), rng.integers(0, n // 3, (1, k))
    neg[0, 4] = pos[1]
    gp = rng.standard_normal((b, 1)).astype(np.float32).astype(np.float64)
    gn = rng.standard_normal((b, k)).astype(np.float32).astype(np.float64)
    opt.zero_grad()
    p_rows = emb(torch.tensor(pos, device="cuda"), "positive_entity")
    n_rows = emb(torch.tensor(neg, device="cuda").view(-1), "negative_entity")
    lp = native_cal_logit(p_rows.unsqueeze(1), t_qs)
    ln = native_cal_logit(n_rows.view(1, k, -1), t_qs)
    assert lp.shape == (b, 1) and ln.shape == (b, k)
    ((lp * torch.tensor(gp, dtype=torch.float32, device="cuda")).sum() +
     (ln * torch.tensor(gn, dtype=torch.float32, device="cuda")).sum()).backward()
    assert len(opt.fused_list) == 2 and not opt.grad_list and opt.stats["materialized_lookups"] == 0
    assert opt.stats["dense_fallbacks"] == 0
    opt.apply_grad(lr)

    neg_full = np.broadcast_to(neg, (b, k))
    o_lp, rows_p = _oracle_branch_logits(name, table, pos.reshape(b, 1), qs, 0.0, 0.0)
    o_ln, rows_n = _oracle_branch_logits(name, table, neg_full, qs, 0.0, 0.0)
    assert_close(lp.detach().cpu().numpy(), o_lp[:, 0], REL_F32, "positive logits")
    assert_close(ln.detach().cpu().numpy(), o_ln[:, 0], REL_F32, "negative logits")
    gr_p, gq_p = _oracle_grads(name, table, pos.reshape(b, 1), qs, rows_p, o_lp, gp, 0.0)
    gr_n, gq_n = _oracle_grads(name, table, neg_full, qs, rows_n, o_ln, gn, 0.0)
    for t, a, c in zip(t_qs, gq_p, gq_n):
        assert_close(t.grad.cpu().numpy(), a + c, REL_F32, "query gradient")
    uniq, inverse, _, _ = orc.merge_indices(np.concatenate([pos.reshape(-1), neg_full.reshape(-1)]))
    merged = orc.merge_grads(np.concatenate([gr_p, gr_n]), inverse, uniq.size)
    w, m, v = table.copy(), np.zeros_like(table), np.zeros_like(table)
    orc.adam_rows(w, m, v, uniq, merged, lr, 1)
    assert_close(emb.state_sum_fo.cpu().numpy()[uniq], m[uniq], REL_F32, "first moment")
    assert_adam_weights(emb.embedding.detach().cpu().numpy(), w, merged, uniq, lr, "weights")


def test_inverse_query_call_sequence_runs_on_the_reverse_layout():
    """Inverse ('<') queries, kg_reasoning.py:306-336: the TAIL entity is looked up and becomes the 'entity' operand
    [B,1,D] (embed_reverse_query, :252-255), while the negatives go through the relation projection
    (cal_reverse_logit, :257-263; vec.py:58-60: rows + relation) and arrive as the 'query' operand [B,1,K,D].
    Arithmetic on the negatives' handle needs their values, and the distance has nothing to gather-fuse: both
    lookups fall back to rows, the operator runs on its reverse-layout kernels, and apply_grad merges the two
    gradient-row records.  Logits, relation gradient and the Adam step against the float64 oracle."""
    from smore_amd.embedding.embed_optimizer import AdamEmbedOptimizer
    from smore_amd.embedding.sparse_embed import SparseEmbedding
    from smore_amd.torchext.ext_ops import l1_dist
    n, d, b, k, lr = 300, 32, 6, 20, 1e-3
    rng = np.random.default_rng(31)
    table = rng.uniform(-0.07, 0.07, (n, d)).astype(np.float32).astype(np.float64)
    rel = rng.uniform(-0.07, 0.07, (b, d)).astype(np.float32).astype(np.float64)
    tail, neg = rng.integers(0, n, b), rng.integers(0, n // 3, (b, k))
    gn = rng.standard_normal((b, k)).astype(np.float32).astype(np.float64)
    emb = SparseEmbedding(n, d).cuda()
    with torch.no_grad():
        emb.embedding.copy_(torch.tensor(table, dtype=torch.float32))
    opt = AdamEmbedOptimizer(types.SimpleNamespace(optim_mode="(aggr,adam,gpu,False,5)", share_optim_stats=True), emb, 0)
    t_rel = torch.tensor(rel, dtype=torch.float32, device="cuda", requires_grad=True)
    gamma = torch.nn.Parameter(torch.Tensor([12.0]).cuda(), requires_grad=False)

    opt.zero_grad()
    all_negative = emb(torch.tensor(neg, device="cuda").view(-1), "negative_entity")
    inv_query_embed = emb(torch.tensor(tail, device="cuda")).unsqueeze(1)                  # embed_reverse_query
    all_negative.job_handle.sync()
    embedding = [all_negative.view(b, k, -1)]
    embedding = [embedding[0] + t_rel.unsqueeze(1)]                                          # relation_projection
    query_embedding = [e.unsqueeze(1) for e in embedding]
    logit = gamma - l1_dist(inv_query_embed, query_embedding[0])                             # custom_cal_logit, vec.py:85-90
    logit = torch.max(logit, dim=1)[0]
    assert logit.shape == (b, k)
    (logit * torch.tensor(gn, dtype=torch.float32, device="cuda")).sum().backward()
    assert len(opt.grad_list) == 2 and not opt.fused_list
    opt.apply_grad(lr)

    # oracle: dist(entity = tail rows [B,1,D], query = negatives + relation [B,K,D]) -> [B,K]
    e = orc.gather(table, tail).reshape(b, 1, d)
    q = orc.gather(table, neg).reshape(b, k, d) + rel[:, None, :]
    want = 12.0 - orc.dist_forward("l1", e, q)
    assert_close(logit.detach().cpu().numpy(), want, REL_F32, "inverse-query logits")
    g_e, g_q, _ = orc.dist_backward("l1", -gn, e, q)
    assert_close(t_rel.grad.cpu().numpy(), g_q.sum(axis=1), REL_F32, "relation gradient")
    w, m, v, uniq, merged = oracle_adam_step(table, [tail, neg], [g_e.reshape(b, d), g_q.reshape(b * k, d)], lr, 1)
    assert_close(emb.state_sum_fo.cpu().numpy()[uniq], m[uniq], REL_F32, "inverse query: first moment")
    assert_adam_weights(emb.embedding.detach().cpu().numpy(), w, merged, uniq, lr, "inverse query: weights")


@pytest.mark.parametrize("name", list(CASES))
def test_anchor_lookups_join_the_fused_records_in_one_update(name, monkeypatch):
    """Every query of the reference starts from the embedding of its anchor entities: a plain lookup in
    embed_query (box.py:137 and siblings) whose rows feed the query side, so that autograd hands the optimizer
    gradient ROWS for them (embed_optimizer.py:63-66) next to the fused record of positives + negatives.  A
    restated 1p query: queries = f(anchor rows, relation tensors).  The step must stay on the fused entity pass
    (no gradient rows materialised for the scored pairs, one plan, one update per entity -- also for entities
    that are anchor and negative at once); logits, relation gradients and Adam state against the oracle."""
    from smore_amd import fused
    from smore_amd.embedding.embed_optimizer import AdamEmbedOptimizer
    from smore_amd.embedding.sparse_embed import SparseEmbedding

    def no_gradient_rows(*a, **k):
        raise AssertionError("the scored pairs must not go through materialised gradient rows")
    monkeypatch.setattr(fused, "rows_backward", no_gradient_rows)
    cls, extra, model, n_q, mul, gamma, cen = CASES[name]
    n, d, b, k, lr = 300, 32, 6, 24, 1e-3
    rng = np.random.default_rng(23)
    f32 = lambda a: np.asarray(a).astype(np.float32).astype(np.float64)
    table, _ = _table_and_queries(name, n, d, b, 1, rng)
    if name.startswith("beta"):
        rel = [f32(rng.uniform(0.5, 1.5, (b, d))) for _ in range(2)]           # positive scales keep alpha, beta > 0
    else:
        rel = [f32(rng.uniform(-0.07, 0.07, (b, d))) for _ in range(n_q)]
        if name in ("box", "box_native"):
            rel[1] = np.abs(rel[1])
    emb = SparseEmbedding(n, mul * d).cuda()
    with torch.no_grad():
        emb.embedding.copy_(torch.tensor(table, dtype=torch.float32))
    opt = AdamEmbedOptimizer(types.SimpleNamespace(optim_mode="(aggr,adam,gpu,False,5)", share_optim_stats=True), emb, 0)
    net = cls(emb, gamma, *extra).cuda()
    t_rel = [torch.tensor(r, dtype=torch.float32, device="cuda", requires_grad=True) for r in rel]

    def embed_query(rows, rels, lib):
        """rows [B, mul*d] -> the model's query tensors [B, d] each (lib = torch or numpy)."""
        if name.startswith("beta"):
            rows = lib.clip(rows + 1.0, 0.05, 1e9) if lib is np else torch.clamp(rows + 1.0, 0.05, 1e9)
            return [rows[:, :d] * rels[0], rows[:, d:] * rels[1]]
        if mul == 2:
            return [rows[:, :d] + rels[0], rows[:, d:] + rels[1]]
        return [rows + rels[0]] + list(rels[1:])

    w, m, v = table.copy(), np.zeros_like(table), np.zeros_like(table)
    for step in (1, 2):
        pos = rng.integers(0, n, b)
        neg = rng.integers(0, n // 4, (b, k))
        anchor = rng.integers(0, n // 4, b)                                    # some anchors are negatives too
        anchor[0], anchor[1] = neg[0, 0], anchor[0]
        gp, gn = f32(rng.standard_normal((b, 1))), f32(rng.standard_normal((b, k)))
        opt.zero_grad()
        for t in t_rel:
            t.grad = None
        a_rows = emb(torch.tensor(anchor, device="cuda"), "anchor")
        a_rows.job_handle.sync()
        t_qs = [q.view(b, 1, 1, d) for q in embed_query(a_rows, t_rel, torch)]
        lp, ln = net(torch.tensor(pos, device="cuda"), torch.tensor(neg, device="cuda"), t_qs)
        ((lp * torch.tensor(gp, dtype=torch.float32, device="cuda")).sum() +
         (ln * torch.tensor(gn, dtype=torch.float32, device="cuda")).sum()).backward()
        assert len(opt.fused_list) == 1 and len(opt.grad_list) == 1
        opt.apply_grad(lr)

        qs = [q.reshape(b, 1, 1, d) for q in embed_query(orc.gather(w, anchor), rel, np)]
        o_lp, rows_p = _oracle_branch_logits(name, w, pos.reshape(b, 1), qs, gamma, cen)
        o_ln, rows_n = _oracle_branch_logits(name, w, neg, qs, gamma, cen)
        assert_close(lp.detach().cpu().numpy(), o_lp[:, 0], REL_F32, f"{name} positive logits, step {step}")
        assert_close(ln.detach().cpu().numpy(), o_ln[:, 0], REL_F32, f"{name} negative logits, step {step}")
        gr_p, gq_p = _oracle_grads(name, w, pos.reshape(b, 1), qs, rows_p, o_lp, gp, cen)
        gr_n, gq_n = _oracle_grads(name, w, neg, qs, rows_n, o_ln, gn, cen)
        gq = [(a + c).reshape(b, d) for a, c in zip(gq_p, gq_n)]              # d loss / d query tensors
        raw = orc.gather(w, anchor)
        if name.startswith("beta"):
            reg = np.clip(raw + 1.0, 0.05, 1e9)
            mask = (raw + 1 >= 0.05) & (raw + 1 <= 1e9)
            g_anchor = np.concatenate([gq[0] * rel[0], gq[1] * rel[1]], axis=1) * mask
            g_rel = [gq[0] * reg[:, :d], gq[1] * reg[:, d:]]
        elif mul == 2:
            g_anchor, g_rel = np.concatenate(gq, axis=1), gq
        else:
            g_anchor, g_rel = gq[0], gq
        for t, want in zip(t_rel, g_rel):
            assert_close(t.grad.cpu().numpy(), want, REL_F32, f"{name} relation gradient, step {step}")
        w_before = w.copy()
        w, m, v, uniq, merged = oracle_adam_step(w, [pos, neg, anchor], [gr_p, gr_n, g_anchor], lr, step, m, v)
        got = emb.embedding.detach().cpu().numpy().astype(np.float64)
        touched = np.zeros(n, bool)
        touched[uniq] = True
        assert np.array_equal(got[~touched], w_before[~touched]), "rows outside the step must keep their bits"
        assert_close(emb.state_sum_fo.cpu().numpy()[touched], m[touched], REL_F32, f"{name} first moment, step {step}")
        assert_close(emb.state_sum_sq.cpu().numpy()[touched], v[touched], REL_F32, f"{name} second moment, step {step}")
        assert_adam_weights(got, w, merged, uniq, lr, f"{name} weights, step {step}")
        w = got.copy()   # continue from the device's fp32 weights so that step 2 compares one step, not two


def test_shared_negatives_beside_positives_share_one_update():
    """--share_negative (online_sampler.py:155-157): negatives [1,K] for the whole batch, positives [B] per query,
    both scored by unchanged model code against one branch of queries.  They leave two records with the optimizer
    -- the positives' B pairs and the K shared ids, which are never expanded to [B, K] -- and apply_grad reduces
    both behind ONE plan (an entity that is positive and shared negative gets one update); the is_negative_mat mask
    of train_process.py:195-196 multiplies the negative logits.  Logits, query gradient and the Adam step against
    the oracle."""
    from smore_amd.embedding.embed_optimizer import AdamEmbedOptimizer
    from smore_amd.embedding.sparse_embed import SparseEmbedding
    n, d, b, k, lr = 300, 16, 5, 12, 1e-3
    rng = np.random.default_rng(9)
    f32 = lambda a: np.asarray(a).astype(np.float32).astype(np.float64)
    table = f32(rng.uniform(-0.07, 0.07, (n, d)))
    q = f32(rng.uniform(-0.07, 0.07, (b, 1, 1, d)))
    pos, neg = rng.integers(0, n, b), rng.integers(0, n, (1, k))
    pos[0] = neg[0, 0]                                                       # a positive that is also a shared negative
    mask = (rng.random((b, k)) < 0.8).astype(np.float64)
    gp, gn = f32(rng.standard_normal((b, 1))), f32(rng.standard_normal((b, k)))
    emb = SparseEmbedding(n, d).cuda()
    with torch.no_grad():
        emb.embedding.copy_(torch.tensor(table, dtype=torch.float32))
    opt = AdamEmbedOptimizer(types.SimpleNamespace(optim_mode="(aggr,adam,gpu,False,5)", share_optim_stats=True), emb, 0)
    net = Vec(emb, 12.0, "l1").cuda()
    tq = torch.tensor(q, dtype=torch.float32, device="cuda", requires_grad=True)
    dev = lambda a: torch.tensor(a, dtype=torch.float32, device="cuda")
    opt.zero_grad()
    p_rows = emb(torch.tensor(pos, device="cuda"), "positive_entity")
    n_rows = emb(torch.tensor(neg, device="cuda").view(-1), "negative_entity")
    p_rows.job_handle.sync()
    lp = net.cal_logit(p_rows.unsqueeze(1), None, [tq])
    n_rows.job_handle.sync()
    ln = net.cal_logit(n_rows.view(1, k, -1), None, [tq])
    ln = ln * dev(mask)
    ((lp * dev(gp)).sum() + (ln * dev(gn)).sum()).backward()
    assert sorted(tuple(r["ids"].shape) for r in opt.fused_list) == [(1, k), (b, 1)] and not opt.grad_list
    assert opt.stats["materialized_lookups"] == 0 and opt.stats["dense_fallbacks"] == 0
    opt.apply_grad(lr)
    assert opt.stats["per_record_merges"] == 0

    ids = np.concatenate([pos.reshape(b, 1), np.broadcast_to(neg, (b, k))], axis=1)
    rows = orc.gather(table, ids).reshape(b, 1 + k, d)
    want = orc.score_forward("l1", rows, q[:, 0], None, 12.0)
    assert_close(lp.detach().cpu().numpy(), want[:, :1], REL_F32, "positive logits")
    assert_close(ln.detach().cpu().numpy(), want[:, 1:] * mask, REL_F32, "masked shared-negative logits")
    g_rows, g_q, _ = orc.score_backward("l1", np.concatenate([gp, gn * mask], axis=1), rows, q[:, 0], None)
    assert_close(tq.grad.cpu().numpy()[:, 0], g_q, REL_F32, "query gradient")
    w, m, v, uniq, merged = oracle_adam_step(table, [ids], [g_rows.reshape(b * (1 + k), d)], lr, 1)
    assert_close(emb.state_sum_fo.cpu().numpy()[uniq], m[uniq], REL_F32, "first moment")
    assert_adam_weights(emb.embedding.detach().cpu().numpy(), w, merged, uniq, lr, "weights")


def test_a_lookup_handle_as_the_query_operand():
    """Negatives handed to the operator as its QUERY operand without any arithmetic first (the reverse layout with
    an identity projection): the handle stands for its rows, the operator runs on its reverse-layout kernels and
    the lookup's gradient rows reach the optimizer."""
    from smore_amd.embedding.embed_optimizer import AdamEmbedOptimizer
    from smore_amd.embedding.sparse_embed import SparseEmbedding
    from smore_amd.torchext.ext_ops import l1_dist
    n, d, b, k, lr = 200, 16, 4, 9, 1e-3
    rng = np.random.default_rng(41)
    table = rng.uniform(-0.07, 0.07, (n, d)).astype(np.float32).astype(np.float64)
    tail, neg = rng.integers(0, n, b), rng.integers(0, n, (b, k))
    gn = rng.standard_normal((b, k)).astype(np.float32).astype(np.float64)
    emb = SparseEmbedding(n, d).cuda()
    with torch.no_grad():
        emb.embedding.copy_(torch.tensor(table, dtype=torch.float32))
    opt = AdamEmbedOptimizer(types.SimpleNamespace(optim_mode="(aggr,adam,gpu,False,5)", share_optim_stats=True), emb, 0)
    opt.zero_grad()
    entity = emb(torch.tensor(tail, device="cuda")).unsqueeze(1)
    queries = emb(torch.tensor(neg, device="cuda").view(-1), "negative_entity").view(b, k, -1)
    logit = 12.0 - l1_dist(entity, queries)
    assert logit.shape == (b, k)
    (logit * torch.tensor(gn, dtype=torch.float32, device="cuda")).sum().backward()
    assert len(opt.grad_list) == 2 and not opt.fused_list
    opt.apply_grad(lr)
    e, q = orc.gather(table, tail).reshape(b, 1, d), orc.gather(table, neg).reshape(b, k, d)
    assert_close(logit.detach().cpu().numpy(), 12.0 - orc.dist_forward("l1", e, q), REL_F32, "logits, handle as query")
    g_e, g_q, _ = orc.dist_backward("l1", -gn, e, q)
    w, m, v, uniq, merged = oracle_adam_step(table, [tail, neg], [g_e.reshape(b, d), g_q.reshape(b * k, d)], lr, 1)
    assert_close(emb.state_sum_fo.cpu().numpy()[uniq], m[uniq], REL_F32, "first moment, handle as query")
    assert_adam_weights(emb.embedding.detach().cpu().numpy(), w, merged, uniq, lr, "weights, handle as query")
