"""The sparse-embedding driver protocol (zero_grad -> lookups/scores -> backward -> apply_grad) on the
HIP path, against the CPU oracle's float64 pipeline."""
import types

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests.util import (REL_F32, assert_adam_weights, assert_close, oracle_adam_step, oracle_union_grads,
                        oracle_union_logits)

pytestmark = pytest.mark.gpu


def _setup(n, d, seed):
    from smore_amd.embedding.embed_optimizer import AdamEmbedOptimizer
    from smore_amd.embedding.sparse_embed import SparseEmbedding
    torch.manual_seed(seed)
    emb = SparseEmbedding(n, d).cuda()
    emb.init_params(-0.07, 0.07)
    args = types.SimpleNamespace(optim_mode="(aggr,adam,gpu,False,5)", share_optim_stats=True)
    opt = AdamEmbedOptimizer(args, emb, 0)
    opt.lazy_lookup = False    # these tests use sp_embed(ids) for the plain lookup + dense operators (the lazy route: test_dropin_gpu.py)
    return emb, opt


def test_lookup_and_plain_gradients_match_oracle():
    """positives + negatives through plain lookups and the autograd box operators, one Adam step."""
    from smore_amd.torchext import ext_ops
    n, d, b, k, lr = 300, 32, 6, 9, 1e-3
    emb, opt = _setup(n, d, 1)
    w0 = emb.embedding.detach().cpu().numpy().astype(np.float64)
    rng = np.random.default_rng(2)
    pos = torch.tensor(rng.integers(0, n, b), device="cuda")
    neg = torch.tensor(rng.integers(0, n, (b, k)), device="cuda")
    c = torch.tensor(rng.uniform(-0.07, 0.07, (b, 1, d)), dtype=torch.float32, device="cuda", requires_grad=True)
    o = torch.tensor(np.abs(rng.uniform(-0.07, 0.07, (b, 1, d))), dtype=torch.float32, device="cuda", requires_grad=True)
    gp = torch.tensor(rng.standard_normal((b, 1)), dtype=torch.float32, device="cuda")
    gn = torch.tensor(rng.standard_normal((b, k)), dtype=torch.float32, device="cuda")

    opt.zero_grad()
    rows_p = emb(pos, "positive_entity")
    rows_n = emb(neg.view(-1), "negative_entity")
    assert rows_p.shape == (b, d) and rows_n.shape == (b * k, d)
    rows_p.job_handle.sync()
    assert torch.equal(rows_p, emb.embedding.detach()[pos])

    def logit(rows):
        return 24 - ext_ops.box_dist_out(rows, c, o) - 0.02 * ext_ops.box_dist_in(rows, c, o)

    lp = logit(rows_p.unsqueeze(1))
    ln = logit(rows_n.view(b, k, -1))
    ((lp * gp).sum() + (ln * gn).sum()).backward()
    opt.apply_grad(lr)
    opt.check_ids()

    # oracle: same pipeline in float64
    cn, on = c.detach().cpu().numpy().astype(np.float64), o.detach().cpu().numpy().astype(np.float64)
    gpn, gnn = gp.cpu().numpy().astype(np.float64), gn.cpu().numpy().astype(np.float64)
    pos_n, neg_n = pos.cpu().numpy(), neg.cpu().numpy()
    rp = orc.gather(w0, pos_n).reshape(b, 1, d)
    rn = orc.gather(w0, neg_n).reshape(b, k, d)
    assert_close(lp.detach().cpu().numpy(), orc.score_forward("box", rp, cn, on, 24.0, 0.02), REL_F32, "pos logit")
    assert_close(ln.detach().cpu().numpy(), orc.score_forward("box", rn, cn, on, 24.0, 0.02), REL_F32, "neg logit")
    g_rp, gc_p, go_p = orc.score_backward("box", gpn, rp, cn, on, 0.02)
    g_rn, gc_n, go_n = orc.score_backward("box", gnn, rn, cn, on, 0.02)
    assert_close(c.grad.cpu().numpy(), gc_p + gc_n, REL_F32, "center grad")
    assert_close(o.grad.cpu().numpy(), go_p + go_n, REL_F32, "offset grad")
    all_idx = np.concatenate([pos_n.reshape(-1), neg_n.reshape(-1)])
    all_g = np.concatenate([g_rp.reshape(b, d), g_rn.reshape(b * k, d)])
    uniq, inverse, _, _ = orc.merge_indices(all_idx)
    merged = orc.merge_grads(all_g, inverse, uniq.size)
    w, m, v = w0.copy(), np.zeros_like(w0), np.zeros_like(w0)
    orc.adam_rows(w, m, v, uniq, merged, lr, 1)
    got = emb.embedding.detach().cpu().numpy()
    touched = np.zeros(n, bool)
    touched[uniq] = True
    err = np.abs(got - w)[touched]
    assert (err > 1e-5 * np.maximum(np.abs(w[touched]), 0.04)).mean() < 1e-3 and err.max() < lr
    assert np.array_equal(got[~touched], w0[~touched].astype(np.float32))
    assert_close(emb.state_sum_fo.cpu().numpy()[touched], m[touched], REL_F32, "first moment")


def test_fused_scorer_alone_and_mixed_with_plain_lookup():
    """score_negatives (gather-fused) gives the same step as plain lookups + autograd operators,
    both alone and when a plain positive lookup shares the step."""
    from smore_amd.torchext import ext_ops
    n, d, b, k, lr = 500, 64, 8, 16, 1e-3
    rng = np.random.default_rng(3)
    pos_n = rng.integers(0, n, b)
    neg_n = rng.integers(0, n // 10, (b, k))  # few distinct ids: long segments
    cn = rng.uniform(-0.07, 0.07, (b, 1, d)).astype(np.float32)
    on = np.abs(rng.uniform(-0.07, 0.07, (b, 1, d))).astype(np.float32)
    gp_n = rng.standard_normal((b, 1)).astype(np.float32)
    gn_n = rng.standard_normal((b, k)).astype(np.float32)

    def run(fused_neg, with_pos):
        emb, opt = _setup(n, d, 5)
        c = torch.tensor(cn, device="cuda", requires_grad=True)
        o = torch.tensor(on, device="cuda", requires_grad=True)
        pos, neg = torch.tensor(pos_n, device="cuda"), torch.tensor(neg_n, device="cuda")
        for step in range(2):
            opt.zero_grad()
            c.grad = o.grad = None
            loss = 0
            if with_pos:
                rp = emb(pos, "positive_entity").unsqueeze(1)
                lp = 24 - ext_ops.box_dist_out(rp, c, o) - 0.02 * ext_ops.box_dist_in(rp, c, o)
                loss = loss + (lp * torch.tensor(gp_n, device="cuda")).sum()
            if fused_neg:
                ln = opt.score_negatives("box", neg, c, o, gamma=24.0, cen=0.02)
            else:
                rn = emb(neg.view(-1), "negative_entity").view(b, k, -1)
                ln = 24 - ext_ops.box_dist_out(rn, c, o) - 0.02 * ext_ops.box_dist_in(rn, c, o)
            loss = loss + (ln * torch.tensor(gn_n, device="cuda")).sum()
            loss.backward()
            opt.apply_grad(lr)
        opt.check_ids()
        return (emb.embedding.detach().cpu().numpy(), emb.state_sum_fo.cpu().numpy(), emb.state_sum_sq.cpu().numpy(),
                c.grad.cpu().numpy(), o.grad.cpu().numpy(), ln.detach().cpu().numpy())

    for with_pos in (False, True):
        a = run(True, with_pos)
        r = run(False, with_pos)
        assert_close(a[5], r[5], REL_F32, "logits")
        assert_close(a[3], r[3], REL_F32, "center grad")
        assert_close(a[4], r[4], REL_F32, "offset grad")
        assert_close(a[1], r[1], 5 * REL_F32, "first moment")
        err = np.abs(a[0] - r[0])
        assert (err > 1e-5 * np.maximum(np.abs(r[0]), 0.04)).mean() < 1e-3 and err.max() < 2 * lr


def test_shared_negatives_with_mask_match_the_dense_operators():
    """--share_negative layout: ids [1,K] scored by every query, logits multiplied by the is_negative_mat
    mask (train_process.py:195-196); fused scorer against plain lookup + broadcasting dense operators."""
    from smore_amd.torchext import ext_ops
    n, d, b, k, lr = 400, 48, 7, 33, 1e-3
    rng = np.random.default_rng(11)
    neg_n = rng.integers(0, n, (1, k))
    cn = rng.uniform(-0.07, 0.07, (b, 1, d)).astype(np.float32)
    on = np.abs(rng.uniform(-0.07, 0.07, (b, 1, d))).astype(np.float32)
    mask_n = (rng.random((b, k)) > 0.2).astype(np.float32)
    gn_n = rng.standard_normal((b, k)).astype(np.float32)

    def run(fused_neg):
        emb, opt = _setup(n, d, 7)
        w0.append(emb.embedding.detach().cpu().numpy().astype(np.float64))
        c = torch.tensor(cn, device="cuda", requires_grad=True)
        o = torch.tensor(on, device="cuda", requires_grad=True)
        neg = torch.tensor(neg_n, device="cuda")
        opt.zero_grad()
        if fused_neg:
            ln = opt.score_negatives("box", neg, c, o, gamma=24.0, cen=0.02)
        else:
            rn = emb(neg.view(-1), "negative_entity").view(1, k, -1)      # [1,K,D] against [B,1,D] queries
            ln = 24 - ext_ops.box_dist_out(rn, c, o) - 0.02 * ext_ops.box_dist_in(rn, c, o)
        assert ln.shape == (b, k)
        ((ln * torch.tensor(mask_n, device="cuda")) * torch.tensor(gn_n, device="cuda")).sum().backward()
        opt.apply_grad(lr)
        opt.check_ids()
        return (ln.detach().cpu().numpy(), c.grad.cpu().numpy(), o.grad.cpu().numpy(), emb.state_sum_fo.cpu().numpy(),
                emb.embedding.detach().cpu().numpy())

    w0 = []
    a, r = run(True), run(False)
    for x, y, what in zip(a[:4], r[:4], ("logits", "center grad", "offset grad", "first moment")):
        assert_close(x, y, 5 * REL_F32, what)
    # masked-out pairs still touch their rows: every listed id has moved (momentum), nothing else has
    assert np.abs(a[4] - r[4]).max() < 2 * lr
    # the float64 oracle as the third party: every query scores the K shared rows, the mask multiplies the
    # upstream gradient, masked pairs stay in the merge (their rows are touched with a zero term)
    assert np.array_equal(w0[0], w0[1])
    ids = np.broadcast_to(neg_n, (b, k))
    qs = [cn.astype(np.float64)[:, None], on.astype(np.float64)[:, None]]
    logit, rows = oracle_union_logits("box", w0[0], ids, qs, 24.0, 0.02)
    g_rows, g_qs = oracle_union_grads("box", w0[0], ids, qs, rows, logit, (mask_n * gn_n).astype(np.float64), 0.02)
    w, m, _, uniq, merged = oracle_adam_step(w0[0], [ids], [g_rows], lr, 1)
    for got, route in ((a, "fused"), (r, "dense")):
        assert_close(got[0], logit[:, 0], REL_F32, f"shared negatives, {route}: logits vs oracle")
        assert_close(got[1], g_qs[0][:, 0], REL_F32, f"shared negatives, {route}: center grad vs oracle")
        assert_close(got[2], g_qs[1][:, 0], REL_F32, f"shared negatives, {route}: offset grad vs oracle")
        assert_close(got[3][uniq], m[uniq], REL_F32, f"shared negatives, {route}: first moment vs oracle")
        assert_adam_weights(got[4], w, merged, uniq, lr, f"shared negatives, {route}: weights vs oracle")
        untouched = np.setdiff1d(np.arange(n), uniq)
        assert np.array_equal(got[4][untouched], w0[0][untouched].astype(np.float32))


@pytest.mark.parametrize("model", ["box", "l1", "rotate"])
def test_union_branches_take_the_max_like_custom_cal_logit(model):
    """Union queries [B,U,1,D]: logit = max over the U branches (box.py:163); fused scorer against plain
    lookup + the dense operators' 4-D query form + torch.max.  Only the winning branch gets gradient."""
    from smore_amd.torchext import ext_ops
    n, d, b, u, k, lr = 300, 40, 5, 3, 21, 1e-3
    row = 2 * d if model == "rotate" else d
    rng = np.random.default_rng(5)
    neg_n = rng.integers(0, n, (b, k))
    q1n = rng.uniform(-0.07, 0.07, (b, u, 1, d)).astype(np.float32)
    q2n = np.abs(rng.uniform(-0.07, 0.07, (b, u, 1, d))).astype(np.float32)
    gn_n = rng.standard_normal((b, k)).astype(np.float32)

    def run(fused_neg):
        emb, opt = _setup(n, row, 7)
        w0.append(emb.embedding.detach().cpu().numpy().astype(np.float64))
        q1 = torch.tensor(q1n, device="cuda", requires_grad=True)
        q2 = torch.tensor(q2n, device="cuda", requires_grad=True) if model != "l1" else None
        neg = torch.tensor(neg_n, device="cuda")
        opt.zero_grad()
        if fused_neg:
            ln = opt.score_negatives(model, neg, q1, q2, gamma=24.0, cen=0.02)
        else:
            rn = emb(neg.view(-1), "negative_entity").view(b, k, -1)
            if model == "box":
                ln = 24 - ext_ops.box_dist_out(rn, q1, q2) - 0.02 * ext_ops.box_dist_in(rn, q1, q2)
            elif model == "l1":
                ln = 24 - ext_ops.l1_dist(rn, q1)
            else:
                ln = 24 - ext_ops.rotate_dist(rn, q1, q2)
            assert ln.shape == (b, u, k)
            ln = torch.max(ln, dim=1)[0]
        assert ln.shape == (b, k)
        (ln * torch.tensor(gn_n, device="cuda")).sum().backward()
        opt.apply_grad(lr)
        opt.check_ids()
        grads = [q1.grad.cpu().numpy()] + ([q2.grad.cpu().numpy()] if q2 is not None else [])
        return [ln.detach().cpu().numpy()] + grads + [emb.state_sum_fo.cpu().numpy(), emb.embedding.detach().cpu().numpy()]

    w0 = []
    a, r = run(True), run(False)
    for x, y in zip(a[:-1], r[:-1]):
        assert_close(x, y, 5 * REL_F32, model)
    assert np.abs(a[1]).sum() > 0
    # the float64 oracle as the third party: per-branch logits, max over branches, gradient to the first maximal
    # branch only, one Adam step on the merged rows
    qs = [q1n.astype(np.float64)] + ([q2n.astype(np.float64)] if model != "l1" else [])
    logit, rows = oracle_union_logits(model, w0[0], neg_n, qs, 24.0, 0.02)
    assert len(np.unique(np.argmax(logit, axis=1))) > 1, "the case must have more than one winning branch"
    g_rows, g_qs = oracle_union_grads(model, w0[0], neg_n, qs, rows, logit, gn_n.astype(np.float64), 0.02)
    w, m, _, uniq, merged = oracle_adam_step(w0[0], [neg_n], [g_rows], lr, 1)
    for got, route in ((a, "fused"), (r, "dense")):
        assert_close(got[0], logit.max(axis=1), REL_F32, f"union {model}, {route}: logits vs oracle")
        for t, want in zip(got[1:], g_qs):
            assert_close(t, want, REL_F32, f"union {model}, {route}: query grad vs oracle")
        assert_close(got[-2][uniq], m[uniq], REL_F32, f"union {model}, {route}: first moment vs oracle")
        assert_adam_weights(got[-1], w, merged, uniq, lr, f"union {model}, {route}: weights vs oracle")


def test_positives_as_column_zero_of_the_fused_call():
    """One score_negatives call on [positive | negatives] ids gives both logit blocks and keeps apply_grad on
    its one-record path; same logits, query gradients and table update as a plain positive lookup through
    the dense operators plus a fused call for the negatives (two records merged into one Adam step)."""
    from smore_amd.torchext import ext_ops
    n, d, b, k, lr = 500, 32, 6, 17, 1e-3
    rng = np.random.default_rng(21)
    pos_n, neg_n = rng.integers(0, n, (b, 1)), rng.integers(0, n, (b, k))
    neg_n[0, 0] = pos_n[0, 0]                       # an entity that is both a positive and a negative
    cn = rng.uniform(-0.07, 0.07, (b, 1, d)).astype(np.float32)
    on = np.abs(rng.uniform(-0.07, 0.07, (b, 1, d))).astype(np.float32)
    gp, gn = rng.standard_normal((b, 1)).astype(np.float32), rng.standard_normal((b, k)).astype(np.float32)

    def run(one_call):
        emb, opt = _setup(n, d, 7)
        w0.append(emb.embedding.detach().cpu().numpy().astype(np.float64))
        c = torch.tensor(cn, device="cuda", requires_grad=True)
        o = torch.tensor(on, device="cuda", requires_grad=True)
        pos, neg = torch.tensor(pos_n, device="cuda"), torch.tensor(neg_n, device="cuda")
        opt.zero_grad()
        if one_call:
            logits = opt.score_negatives("box", torch.cat([pos, neg], dim=1), c, o, gamma=24.0, cen=0.02)
            lp, ln = logits[:, :1], logits[:, 1:]
        else:
            rp = emb(pos.view(-1), "positive_entity").unsqueeze(1)
            lp = 24 - ext_ops.box_dist_out(rp, c, o) - 0.02 * ext_ops.box_dist_in(rp, c, o)
            ln = opt.score_negatives("box", neg, c, o, gamma=24.0, cen=0.02)
        ((lp * torch.tensor(gp, device="cuda")).sum() + (ln * torch.tensor(gn, device="cuda")).sum()).backward()
        opt.apply_grad(lr)
        opt.check_ids()
        return [x.detach().cpu().numpy() for x in (lp, ln, c.grad, o.grad, emb.state_sum_fo, emb.state_sum_sq)] + \
            [emb.embedding.detach().cpu().numpy()]

    w0 = []
    a, r = run(True), run(False)
    for x, y, what in zip(a[:6], r[:6], ("positive logit", "negative logits", "center grad", "offset grad", "m", "v")):
        assert_close(x, y, 5 * REL_F32, what)
    assert np.abs(a[6] - r[6]).max() < 2 * lr
    # the float64 oracle as the third party: positives and negatives are two index streams into one merge
    # (embed_optimizer.py:155-163); the entity that is both gets one row update from the sum of both gradients
    ids = np.concatenate([pos_n, neg_n], axis=1)
    qs = [cn.astype(np.float64)[:, None], on.astype(np.float64)[:, None]]
    gout = np.concatenate([gp, gn], axis=1).astype(np.float64)
    logit, rows = oracle_union_logits("box", w0[0], ids, qs, 24.0, 0.02)
    g_rows, g_qs = oracle_union_grads("box", w0[0], ids, qs, rows, logit, gout, 0.02)
    w, m, v, uniq, merged = oracle_adam_step(w0[0], [ids], [g_rows], lr, 1)
    for got, route in ((a, "one call"), (r, "two records")):
        assert_close(got[0], logit[:, 0, :1], REL_F32, f"positives, {route}: positive logit vs oracle")
        assert_close(got[1], logit[:, 0, 1:], REL_F32, f"positives, {route}: negative logits vs oracle")
        assert_close(got[2], g_qs[0][:, 0], REL_F32, f"positives, {route}: center grad vs oracle")
        assert_close(got[3], g_qs[1][:, 0], REL_F32, f"positives, {route}: offset grad vs oracle")
        assert_close(got[4][uniq], m[uniq], REL_F32, f"positives, {route}: first moment vs oracle")
        assert_close(got[5][uniq], v[uniq], REL_F32, f"positives, {route}: second moment vs oracle")
        assert_adam_weights(got[6], w, merged, uniq, lr, f"positives, {route}: weights vs oracle")


def test_step_counter_and_empty_steps():
    emb, opt = _setup(50, 8, 7)
    opt.zero_grad()
    opt.apply_grad(1e-3)  # no gradients: the counter still advances (embed_optimizer.py:156-158)
    assert opt.step == 1
    w0 = emb.embedding.detach().clone()
    opt.zero_grad()
    rows = emb(torch.tensor([3, 3, 7], device="cuda"), "x")
    (rows.sum() * 2.0).backward()
    opt.apply_grad(1e-2)
    assert opt.step == 2
    w = emb.embedding.detach()
    changed = (w != w0).any(dim=1).nonzero().flatten().tolist()
    assert changed == [3, 7]
    # bias correction uses the global step (2), not the row's own first touch
    g = np.array([4.0, 2.0])  # row 3 was looked up twice
    m1, v1 = 0.1 * g, 0.001 * g * g
    want = -1e-2 / (1 - 0.9 ** 2) * m1 / (np.sqrt(v1) / np.sqrt(1 - 0.999 ** 2) + 1e-8)
    got = (w - w0)[[3, 7], 0].cpu().numpy()
    assert np.allclose(got, want, rtol=1e-4)


def test_out_of_range_lookup_is_reported():
    emb, opt = _setup(20, 8, 9)
    opt.zero_grad()
    emb(torch.tensor([1, 25], device="cuda"), "x")
    with pytest.raises(IndexError):
        opt.check_ids()


def test_out_of_range_id_in_a_step_raises_when_the_next_step_begins():
    """The per-step check does not wait for the device: the flag of step n is read where step n+1 passes by -- its
    zero_grad if the flag has landed by then, its apply_grad at the latest (before that update is applied; also an
    apply_grad without gradients), or saving the table.  The bad pair itself updates no row (its key sorts behind
    every real segment)."""
    emb, opt = _setup(20, 8, 9)
    c = torch.zeros(2, 1, 8, device="cuda", requires_grad=True)
    o = torch.ones(2, 1, 8, device="cuda", requires_grad=True)
    w0 = emb.embedding.detach().clone()

    def step(ids):
        ln = opt.score_negatives("box", torch.tensor(ids, device="cuda"), c, o, gamma=1.0, cen=0.02)
        ln.sum().backward()
        opt.apply_grad(1e-3)

    opt.zero_grad()
    step([[1, 25], [2, 3]])
    with pytest.raises(IndexError):
        opt.zero_grad()
        step([[4, 5], [6, 7]])
    changed = (emb.embedding.detach() != w0).any(dim=1).nonzero().flatten().tolist()
    assert changed == [1, 2, 3], "the step that finds the flag raised is not applied"
    opt.zero_grad()       # the flag was cleared when the error was raised
    step([[4, 5], [6, 7]])
    changed = (emb.embedding.detach() != w0).any(dim=1).nonzero().flatten().tolist()
    assert changed == [1, 2, 3, 4, 5, 6, 7]
    opt.check_ids()
    # the other places a waiting flag is looked at: an apply_grad with nothing to apply, and saving the table
    for look in (lambda: opt.apply_grad(1e-3), lambda: emb.state_dict()):
        opt.zero_grad()
        step([[1, 2], [3, 99]])
        with pytest.raises(IndexError):
            look()
    # check_ids_synchronously: the step that met the id fails itself
    opt.check_ids_synchronously = True
    opt.zero_grad()
    with pytest.raises(IndexError):
        step([[1, 2], [3, 99]])


def test_trainer_set_up_protocol_and_cpu_statistics_mode():
    """get_optim_class(args).prepare_optimizers(args, embeds) before the optimizer objects exist (the trainer's
    order, embed_optimizer.py:102-110), the reference scripts' optim_mode with 'cpu' statistics and a squeezed
    second moment, and a lookup with [B,K] ids keeping its shape."""
    from smore_amd.embedding.embed_optimizer import AdamEmbedOptimizer, get_optim_class
    from smore_amd.embedding.sparse_embed import SparseEmbedding
    emb = SparseEmbedding(30, 8).cuda()
    args = types.SimpleNamespace(optim_mode="(aggr, adam, cpu, True, 5)", share_optim_stats=True)
    cls = get_optim_class(args)
    assert cls is AdamEmbedOptimizer
    cls.prepare_optimizers(args, [emb])
    assert emb.state_sum_fo.shape == (30, 8) and emb.state_sum_sq.shape == (30, 1) and emb.state_sum_sq.is_cuda
    fo = emb.state_sum_fo
    opt = cls(args, emb, 0)
    assert emb.state_sum_fo is fo and opt.squeeze and opt.optimizer_device == "cpu"
    opt.lazy_lookup = False
    rows = emb(torch.tensor([[1, 2, 3], [4, 5, 6]], device="cuda"), "x")
    assert rows.shape == (2, 3, 8) and torch.equal(rows[1, 2], emb.embedding.detach()[6])


def test_scoring_without_gradients_saves_no_codes_and_leaves_no_record(monkeypatch):
    """Evaluation on sampled negatives (train_process.py:103-108) runs the model code under torch.no_grad():
    same logits, no sign-code buffer, nothing for apply_grad."""
    from smore_amd import fused
    emb, opt = _setup(60, 16, 13)
    c = torch.rand(4, 1, 16, device="cuda") * 0.1
    o = torch.rand(4, 1, 16, device="cuda") * 0.1
    ids = torch.randint(0, 60, (4, 9), device="cuda")
    opt.zero_grad()
    want = opt.score_negatives("box", ids, c, o, gamma=24.0, cen=0.02)
    made = []
    real = fused.new_codes
    monkeypatch.setattr(fused, "new_codes", lambda *a, **k: made.append(1) or real(*a, **k))
    with torch.no_grad():
        got = opt.score_negatives("box", ids, c, o, gamma=24.0, cen=0.02)
    assert torch.equal(got, want) and not made and not got.requires_grad
    opt.zero_grad()
    opt.apply_grad(1e-3)


def test_state_buffers_are_in_the_state_dict():
    emb, _ = _setup(20, 8, 11)
    sd = emb.state_dict()
    assert {"embedding", "state_sum_fo", "state_sum_sq"} <= set(sd)


def test_checkpoint_round_trip_resumes_the_same_trajectory():
    """model.state_dict() carries the table and the optimizer moments under the reference's names
    (train_process.py:252-262 saves exactly that); a fresh module that loads it continues bit for bit."""
    import io
    n, d, b, k, lr = 200, 16, 4, 12, 1e-3
    rng = np.random.default_rng(8)
    ids = [torch.tensor(rng.integers(0, n, (b, k)), device="cuda") for _ in range(3)]
    c = torch.tensor(rng.uniform(-0.07, 0.07, (b, 1, d)), dtype=torch.float32, device="cuda")
    o = torch.tensor(np.abs(rng.uniform(-0.07, 0.07, (b, 1, d))), dtype=torch.float32, device="cuda")
    g = torch.tensor(rng.standard_normal((b, k)), dtype=torch.float32, device="cuda")

    def train(emb, opt, steps):
        for i in steps:
            opt.zero_grad()
            (opt.score_negatives("box", ids[i], c, o, gamma=24.0, cen=0.02) * g).sum().backward()
            opt.apply_grad(lr)

    emb, opt = _setup(n, d, 5)
    train(emb, opt, [0, 1])
    blob = io.BytesIO()
    torch.save({"model_state_dict": emb.state_dict()}, blob)
    train(emb, opt, [2])

    emb2, opt2 = _setup(n, d, 99)                      # different initial values, overwritten by the load
    blob.seek(0)
    missing, unexpected = emb2.load_state_dict(torch.load(blob, weights_only=True)["model_state_dict"], strict=False)
    assert not missing and not unexpected
    opt2.step = 2                                      # the step counter lives with the trainer, as in the reference
    train(emb2, opt2, [2])
    for name in ("embedding", "state_sum_fo", "state_sum_sq"):
        assert torch.equal(emb.state_dict()[name], emb2.state_dict()[name]), name


@pytest.mark.parametrize("name", ["adam", "sgd", "adagrad", "rmsprop"])
@pytest.mark.parametrize("squeeze", [False, True])
def test_row_optimizers_match_oracle(name, squeeze):
    """Every optimizer of the reference (and its squeezed second moment), three steps of plain lookups."""
    from smore_amd.embedding import embed_optimizer as eo
    from smore_amd.embedding.sparse_embed import SparseEmbedding
    torch.manual_seed(3)
    n, d, lr = 120, 24, 1e-2
    emb = SparseEmbedding(n, d).cuda()
    emb.init_params(-0.5, 0.5)
    args = types.SimpleNamespace(optim_mode=f"(aggr,{name},gpu,{squeeze},5)", share_optim_stats=True)
    opt = eo.get_optim_class(args)(args, emb, 0)
    assert opt.squeeze == squeeze
    w = emb.embedding.detach().cpu().numpy().astype(np.float64)
    m = np.zeros_like(w)
    v = np.zeros((n, 1)) if squeeze else np.zeros_like(w)
    rng = np.random.default_rng(4)
    for step in range(1, 4):
        ids = rng.integers(0, n, 80)
        coef = rng.standard_normal((80, d))
        opt.zero_grad()
        rows = emb(torch.tensor(ids, device="cuda"), "x")
        (rows * torch.tensor(coef, dtype=torch.float32, device="cuda")).sum().backward()
        opt.apply_grad(lr)
        uniq, inverse, _, _ = orc.merge_indices(ids)
        merged = orc.merge_grads(coef.astype(np.float32).astype(np.float64), inverse, uniq.size)
        if name == "adam":
            orc.adam_rows(w, m, v, uniq, merged, lr, step, squeeze=squeeze)
        elif name == "sgd":
            orc.sgd_rows(w, uniq, merged, lr)
        elif name == "adagrad":
            orc.adagrad_rows(w, v, uniq, merged, lr, squeeze=squeeze)
        else:
            orc.rmsprop_rows(w, v, uniq, merged, lr, squeeze=squeeze)
    assert_close(emb.embedding.detach().cpu().numpy(), w, 2e-5, f"{name} weights")
    if name != "sgd":
        state = emb.state_sum_sq if name == "adam" else emb.state_sum
        assert state.shape == ((n, 1) if squeeze else (n, d))
        assert_close(state.cpu().numpy(), v, 2e-5, f"{name} second moment")
    if name == "adam":
        assert_close(emb.state_sum_fo.cpu().numpy(), m, 2e-5, "adam first moment")


@pytest.mark.parametrize("gamma_b", [12.0, 9.0])
def test_fused_records_of_two_query_batches_and_a_plain_lookup_in_one_step(gamma_b):
    """Two score_negatives calls against DIFFERENT query tensors: their records still share one plan and one entity
    pass (each source reads its own stretch of the query rows, laid one batch after the other), together with the
    plain lookup's gradient rows (embed_optimizer.py:155-163), and every entity gets one update.  Against the
    oracle's merge of all three index streams.  Records scored with different margins (second case) cannot share a
    pass: each is reduced to per-entity gradient rows first and those are merged."""
    n, d, b, k, lr = 300, 32, 6, 10, 1e-3
    rng = np.random.default_rng(12)
    f32 = lambda a: np.asarray(a).astype(np.float32).astype(np.float64)
    emb, opt = _setup(n, d, 9)
    table = emb.embedding.detach().cpu().numpy().astype(np.float64)
    qa, qb = f32(rng.uniform(-0.07, 0.07, (b, d))), f32(rng.uniform(-0.07, 0.07, (b, d)))
    ids_a, ids_b = rng.integers(0, n // 3, (b, k)), rng.integers(0, n // 3, (b, k))
    looked = rng.integers(0, n // 3, b)
    ga, gb = f32(rng.standard_normal((b, k))), f32(rng.standard_normal((b, k)))
    gl = f32(rng.standard_normal((b, d)))
    dev = lambda a: torch.tensor(a, dtype=torch.float32, device="cuda")
    ta, tb = dev(qa).requires_grad_(), dev(qb).requires_grad_()
    opt.zero_grad()
    la = opt.score_negatives("l1", torch.tensor(ids_a, device="cuda"), ta, None, gamma=12.0)
    lb = opt.score_negatives("l1", torch.tensor(ids_b, device="cuda"), tb, None, gamma=gamma_b)
    rows = emb(torch.tensor(looked, device="cuda"), "anchor")
    ((la * dev(ga)).sum() + (lb * dev(gb)).sum() + (rows * dev(gl)).sum()).backward()
    assert len(opt.fused_list) == 2 and len(opt.grad_list) == 1
    opt.apply_grad(lr)
    opt.check_ids()
    assert opt.stats["per_record_merges"] == (0 if gamma_b == 12.0 else 2)
    grads = []
    for ids, q, g, t, logit, gamma in ((ids_a, qa, ga, ta, la, 12.0), (ids_b, qb, gb, tb, lb, gamma_b)):
        e = orc.gather(table, ids).reshape(b, k, d)
        assert_close(logit.detach().cpu().numpy(), orc.score_forward("l1", e, q[:, None], None, gamma), REL_F32, "logits")
        g_rows, g_q, _ = orc.score_backward("l1", g, e, q[:, None], None)
        assert_close(t.grad.cpu().numpy(), g_q[:, 0], REL_F32, "query gradient")
        grads.append(g_rows.reshape(b * k, d))
    w, m, v, uniq, merged = oracle_adam_step(table, [ids_a, ids_b, looked], grads + [gl], lr, 1)
    assert_close(emb.state_sum_fo.cpu().numpy()[uniq], m[uniq], REL_F32, "first moment")
    assert_close(emb.state_sum_sq.cpu().numpy()[uniq], v[uniq], REL_F32, "second moment", rms_floor=False)
    assert_adam_weights(emb.embedding.detach().cpu().numpy(), w, merged, uniq, lr, "weights")
