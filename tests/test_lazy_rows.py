"""Host logic of the lazy lookup handle (smore_amd/embedding/lazy_rows.py), no GPU: which call sequences stay
lazy and reach the fused scorer as ONE request with the right model / margin / coefficient / prologue, and which
fall back to the looked-up rows.  The optimizer is replaced by a recorder whose scorer evaluates textbook torch
expressions, so every result is also checked by value."""
import types

import pytest
import torch

from smore_amd.embedding.lazy_rows import LazyLogit, LazyRows
from smore_amd.torchext import ext_ops


class RecordingOptimizer:
    """Stands where EmbeddingOptimizer stands for a LazyRows handle: the real request / batching logic, with the
    launch of the fused scorer replaced by textbook torch expressions and a record of what was asked."""
    from smore_amd.embedding.embed_optimizer import EmbeddingOptimizer as _Real
    lazy_request = _Real.lazy_request
    score_lazy = _Real.score_lazy
    evaluate_pending = _Real.evaluate_pending

    def __init__(self, n, row):
        g = torch.Generator().manual_seed(5)
        table = torch.rand((n, row), generator=g) * 2 - 0.5
        self.sparse_embed = types.SimpleNamespace(embedding=table, dummy_job=types.SimpleNamespace(sync=lambda: None))
        self.scored, self.looked_up, self.pending_scores = [], [], []

    def lookup_rows(self, ids, name=None, for_handle=False):
        self.looked_up.append(name)
        return self.sparse_embed.embedding[ids]

    def _score_max(self, model, ids, q1, q2, gamma, cen, reg):
        logit = self._score_branches(model, ids, q1, q2, gamma, cen, reg)
        return (logit[:, 0], None) if logit.shape[1] == 1 else torch.max(logit, dim=1)

    def _score_branches(self, model, ids, q1, q2, gamma, cen, reg):
        """[B, U, K] logits, as the real optimizer's launch returns them."""
        self.scored.append((model, tuple(ids.shape), gamma, cen, reg))
        e = self.sparse_embed.embedding[ids]
        if reg == "unit_halves":
            re, im = torch.chunk(e, 2, dim=-1)
            e = torch.cat((re / re.norm(dim=-1, keepdim=True), im / im.norm(dim=-1, keepdim=True)), dim=-1)
        elif reg == "unit_row":
            e = e / e.norm(dim=-1, keepdim=True)
        elif reg is not None:
            e = torch.clamp(e + reg[0], reg[1], reg[2])
        if q1.dim() == 3:
            q1, q2 = q1.unsqueeze(1), None if q2 is None else q2.unsqueeze(1)
        sign = 1.0 if model in ("complex", "distmult") else -1.0
        return gamma + sign * _textbook(model, e, (q1, q2), cen)


def _textbook(model, e, queries, cen):
    """dist(e [B,K,row], q [B,U,1,D]) -> [B,U,K] from the definitions of the naive twins (box_dist.py:78-89,
    l1_dist.py:65-67, rotate_dist.py:68-75)."""
    e = e.unsqueeze(1)
    if model == "l1":
        return (e - queries[0]).abs().sum(-1)
    if model == "l2":
        return ((e - queries[0]) ** 2).sum(-1).sqrt()
    if model == "box":
        delta = (e - queries[0]).abs()
        return torch.relu(delta - queries[1]).sum(-1) + cen * torch.minimum(delta, queries[1]).sum(-1)
    if model == "rotate":
        re, im = torch.chunk(e, 2, dim=-1)
        return torch.sqrt((re - queries[0]) ** 2 + (im - queries[1]) ** 2).sum(-1)
    if model == "complex":
        re, im = torch.chunk(e, 2, dim=-1)
        return (re * queries[0] + im * queries[1]).sum(-1)
    if model == "distmult":
        return (e * queries[0]).sum(-1)
    if model == "beta_kl":
        ea, eb = torch.chunk(e, 2, dim=-1)
        D = torch.distributions
        ea, eb, qa, qb = torch.broadcast_tensors(ea, eb, queries[0], queries[1])
        return D.kl.kl_divergence(D.Beta(ea, eb), D.Beta(qa, qb)).sum(-1)
    raise AssertionError(model)


def _queries(b, u, d, n_q, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.rand((b, u, 1, d), generator=g) for _ in range(n_q)]


def test_box_logit_of_the_model_code_is_one_fused_request():
    """box.py:157-164 on the handle of kg_reasoning.py:301-307,349-355."""
    n, d, b, k, u = 50, 8, 3, 5, 2
    opt = RecordingOptimizer(n, d)
    ids = torch.randint(0, n, (b, k), generator=torch.Generator().manual_seed(1))
    gamma = torch.nn.Parameter(torch.tensor([24.0]), requires_grad=False)
    c, o = _queries(b, u, d, 2, 2)
    rows = LazyRows(opt, ids.view(-1), "negative_entity")
    rows.job_handle.sync()
    rows = rows.view(b, k, -1)
    assert isinstance(rows, LazyRows) and rows.shape == (b, k, d)
    d1 = ext_ops.box_dist_out(rows, c, o)
    d2 = ext_ops.box_dist_in(rows, c, o)
    logit = gamma - d1 - 0.02 * d2
    assert isinstance(logit, LazyLogit) and logit.shape == (b, u, k) and not opt.scored
    out, which = torch.max(logit, dim=1)
    assert out.shape == (b, k) and not opt.scored, "the maximum over the branches waits for its first use"
    e = opt.sparse_embed.embedding[ids]
    want, want_which = torch.max(24.0 - _textbook("box", e, (c, o), 0.02), dim=1)
    assert torch.allclose(out, want, rtol=0, atol=1e-5)
    assert opt.scored == [("box", (b, k), 24.0, 0.02, None)] and not opt.looked_up
    assert torch.equal(which.materialize(), want_which)


@pytest.mark.parametrize("op,model,n_q", [("l1_dist", "l1", 1), ("l2_dist", "l2", 1), ("rotate_dist", "rotate", 2)])
def test_one_distance_models(op, model, n_q):
    """vec.py:85-90 and rotate.py:137-142; positives come as [B] ids, unsqueezed to [B,1,row]."""
    n, d, b = 40, 6, 4
    mul = 2 if model == "rotate" else 1
    opt = RecordingOptimizer(n, d * mul)
    ids = torch.arange(b) * 3
    q = _queries(b, 1, d, n_q, 3)
    rows = LazyRows(opt, ids, "positive_entity").unsqueeze(1)
    logit = 12.0 - getattr(ext_ops, op)(rows, *q)
    out = torch.max(logit, dim=1)[0]
    assert not opt.scored, "one branch: the logits wait until somebody needs them"
    assert out.shape == (b, 1) and out.dim() == 2
    assert torch.allclose(out, (12.0 - _textbook(model, opt.sparse_embed.embedding[ids].unsqueeze(1), q, 0.0))[:, 0], rtol=0, atol=1e-5)
    assert opt.scored == [(model, (b, 1), 12.0, 0.0, None)]
    e = opt.sparse_embed.embedding[ids].unsqueeze(1)
    assert torch.allclose(out, (12.0 - _textbook(model, e, q, 0.0))[:, 0], rtol=0, atol=1e-5)


def test_regularizer_becomes_the_prologue_only_for_beta():
    """modules.py:29-36: clamp(rows + base_add, lo, hi) is carried by the handle; a model whose fused scorer has
    no prologue gets the dense route with the regularized rows."""
    n, d, b, k = 30, 4, 2, 3
    opt = RecordingOptimizer(n, 2 * d)
    ids = torch.randint(0, n, (b * k,), generator=torch.Generator().manual_seed(4))
    rows = torch.clamp(LazyRows(opt, ids, "negative_entity").view(b, k, -1) + 1.0, 0.05, 1e9)
    assert isinstance(rows, LazyRows) and rows.reg == (1.0, 0.05, 1e9)
    val = rows.materialize()
    assert torch.equal(val, torch.clamp(opt.sparse_embed.embedding[ids].view(b, k, -1) + 1.0, 0.05, 1e9))
    lazy = ext_ops.beta_kl(rows, ext_ops.BetaDist(*_queries(b, 1, d, 2, 5)))
    assert isinstance(lazy, LazyLogit)
    # an operator without a prologue in the fused scorer: the request is refused by score_lazy's caller contract
    opt1 = RecordingOptimizer(n, d)
    r1 = torch.clamp(LazyRows(opt1, ids, None).view(b, k, -1) + 1.0, 0.05, 1e9)
    assert isinstance(ext_ops.l1_dist(r1, _queries(b, 1, d, 1, 6)[0]), LazyLogit)


class _Normalizer:                  # common/modules.py:38-40
    def __call__(self, embedding):
        return torch.nn.functional.normalize(embedding, p=2, dim=-1)


def _complex_logit(embed_norm, entity_embedding, query_embedding):
    """custom_cal_logit of models/complex.py:140-148 in its 'norm' mode."""
    query_re_embedding, query_im_embedding = query_embedding
    entity_re_embedding, entity_im_embedding = torch.chunk(entity_embedding, 2, dim=-1)
    entity_re_embedding, entity_im_embedding = embed_norm(entity_re_embedding), embed_norm(entity_im_embedding)
    entity_embedding = torch.cat((entity_re_embedding, entity_im_embedding), dim=-1).contiguous()
    logit = ext_ops.complex_sim(entity_embedding, query_re_embedding, query_im_embedding)
    return entity_embedding, torch.max(logit, dim=1)[0]


@pytest.mark.parametrize("branches", [1, 2])
def test_unit_length_halves_of_complex_stay_on_the_handle(branches):
    """chunk / F.normalize / cat of models/complex.py:142-146: the rows are never looked up, the scorer gets ONE
    request for the complex model with the unit-length option, and the value is that of the torch expression."""
    n, d, b, k = 40, 6, 3, 5
    opt = RecordingOptimizer(n, 2 * d)
    ids = torch.randint(0, n, (b * k,), generator=torch.Generator().manual_seed(9))
    qs = _queries(b, branches, d, 2, 12)
    handle = LazyRows(opt, ids, "negative_entity").view(b, k, -1)
    ent, logit = _complex_logit(_Normalizer(), handle, qs)
    assert isinstance(ent, LazyRows) and ent.reg == "unit_halves"
    rows = opt.sparse_embed.embedding[ids].view(b, k, -1)
    F = torch.nn.functional
    re, im = torch.chunk(rows, 2, dim=-1)
    want = torch.max((F.normalize(re, p=2, dim=-1).unsqueeze(1) * qs[0] + F.normalize(im, p=2, dim=-1).unsqueeze(1) * qs[1]).sum(-1), dim=1)[0]
    torch.testing.assert_close(logit + 0.0, want, rtol=1e-6, atol=1e-6)       # (the first use scores the placeholder)
    assert opt.looked_up == [] and opt.scored == [("complex", (b, k), 0.0, 0.0, "unit_halves")]
    # the values the handle stands for, when something else asks for them
    assert torch.equal(ent.materialize(), torch.cat((F.normalize(re, p=2, dim=-1), F.normalize(im, p=2, dim=-1)), dim=-1))


def test_halves_put_to_any_other_use_become_tensors():
    n, d, b, k = 40, 6, 3, 5
    F = torch.nn.functional
    ids = torch.randint(0, n, (b * k,), generator=torch.Generator().manual_seed(10))
    opt = RecordingOptimizer(n, 2 * d)
    rows = opt.sparse_embed.embedding[ids].view(b, k, -1)
    re, im = torch.chunk(rows, 2, dim=-1)
    handle = LazyRows(opt, ids, None).view(b, k, -1)
    h_re, h_im = torch.chunk(handle, 2, dim=-1)
    assert h_re.shape == re.shape and h_im.dim() == 3 and opt.looked_up == []
    # Identity in the place of the normalizer (complex.py:91): the two halves put together are the handle again
    assert torch.cat((h_re, h_im), dim=-1) is handle
    # the halves the other way round, another norm, another axis, one half alone, arithmetic: the tensor's results
    assert torch.equal(torch.cat((h_im, h_re), dim=-1), torch.cat((im, re), dim=-1))
    assert torch.equal(F.normalize(h_re, p=1, dim=-1), F.normalize(re, p=1, dim=-1))
    assert torch.equal(F.normalize(h_re, p=2, dim=1), F.normalize(re, p=2, dim=1))
    assert torch.equal(torch.cat((F.normalize(h_re, p=2, dim=-1), h_im), dim=-1), torch.cat((F.normalize(re, p=2, dim=-1), im), dim=-1))
    assert torch.equal(F.normalize(h_im, p=2, dim=-1) * 2.0, F.normalize(im, p=2, dim=-1) * 2.0)
    assert torch.equal(h_re + 1.0, re + 1.0) and torch.equal(h_im[0], im[0])
    assert len(opt.looked_up) == 1, "one lookup per handle family"
    # three chunks, or chunks along another axis, are no halves
    three = torch.chunk(LazyRows(opt, ids, None).view(b, k, -1), 3, dim=-1)
    assert all(isinstance(t, torch.Tensor) for t in three) and torch.equal(three[1], torch.chunk(rows, 3, dim=-1)[1])
    # unit-length halves under a model that has no such form: dense route, right values
    ent = torch.cat((F.normalize(h_re, p=2, dim=-1), F.normalize(h_im, p=2, dim=-1)), dim=-1)
    q = _queries(b, 1, 2 * d, 1, 3)[0]
    lazy = 12.0 - ext_ops.l1_dist(ent, q)
    assert lazy._fusable() == ("l1", 0.0)      # the expression has the model's form; the request is what is refused:
    assert opt.lazy_request("l1", ent, (q,), 12.0, 0.0) is None and opt.score_lazy("l1", ent, (q,), 12.0, 0.0) is None


def _native_box(gamma, cen, entity_embedding, query_embedding):
    """native_cal_logit of models/box.py:147-155"""
    F = torch.nn.functional
    query_center_embedding, query_offset_embedding = query_embedding
    delta = (entity_embedding.unsqueeze(1) - query_center_embedding).abs()
    distance_out = F.relu(delta - query_offset_embedding)
    distance_in = torch.min(delta, query_offset_embedding)
    logit = gamma - torch.norm(distance_out, p=1, dim=-1) - cen * torch.norm(distance_in, p=1, dim=-1)
    return torch.max(logit, dim=1)[0]


def _native_vec(gamma, cen, entity_embedding, query_embedding):
    """native_cal_logit of models/vec.py:78-83"""
    distance = entity_embedding.unsqueeze(1) - query_embedding[0]
    logit = gamma - torch.norm(distance, p=1, dim=-1)
    return torch.max(logit, dim=1)[0]


def _native_rotate(gamma, cen, entity_embedding, query_embedding):
    """native_cal_logit of models/rotate.py:125-135"""
    query_re_embedding, query_im_embedding = query_embedding
    entity_re_embedding, entity_im_embedding = torch.chunk(entity_embedding.unsqueeze(1), 2, dim=-1)
    re_distance = entity_re_embedding - query_re_embedding
    im_distance = entity_im_embedding - query_im_embedding
    distance = torch.stack([re_distance, im_distance], dim=0)
    distance = distance.norm(dim=0)
    logit = gamma - distance.sum(dim=-1)
    return torch.max(logit, dim=1)[0]


def _native_distmult(gamma, cen, entity_embedding, query_embedding, embed_norm=None):
    """native_cal_logit of models/distmult.py:126-133"""
    entity_embedding = entity_embedding.unsqueeze(1)
    if embed_norm is not None:
        entity_embedding = embed_norm(entity_embedding)
    logit = (query_embedding[0] * entity_embedding).sum(-1)
    return torch.max(logit, dim=1)[0]


def _native_distmult_norm(gamma, cen, entity_embedding, query_embedding):
    return _native_distmult(gamma, cen, entity_embedding, query_embedding, _Normalizer())


def _native_complex(gamma, cen, entity_embedding, query_embedding, embed_norm=None):
    """native_cal_logit of models/complex.py:169-177, the branch for rows of the queries' own batch"""
    query_re_embedding, query_im_embedding = query_embedding
    entity_re_embedding, entity_im_embedding = torch.chunk(entity_embedding.unsqueeze(1), 2, dim=-1)
    if embed_norm is not None:
        entity_re_embedding, entity_im_embedding = embed_norm(entity_re_embedding), embed_norm(entity_im_embedding)
    assert entity_re_embedding.shape[0] == query_re_embedding.shape[0]
    logit = (entity_re_embedding * query_re_embedding + entity_im_embedding * query_im_embedding).sum(dim=-1)
    return torch.max(logit, dim=1)[0]


def _native_complex_norm(gamma, cen, entity_embedding, query_embedding):
    return _native_complex(gamma, cen, entity_embedding, query_embedding, _Normalizer())


@pytest.mark.parametrize("body,model,reg", [(_native_distmult, "distmult", None), (_native_complex, "complex", None),
                                            (_native_complex_norm, "complex", "unit_halves"),
                                            (_native_distmult_norm, "distmult", "unit_row")])
@pytest.mark.parametrize("branches", [1, 2])
def test_native_similarity_bodies_become_one_fused_request(body, model, reg, branches):
    n, d, b, k = 40, 6, 3, 5
    mul = 2 if model == "complex" else 1
    opt = RecordingOptimizer(n, mul * d)
    ids = torch.randint(0, n, (b * k,), generator=torch.Generator().manual_seed(31))
    qs = _queries(b, branches, d, mul, 32)
    logit = body(None, 0.0, LazyRows(opt, ids, "negative_entity").view(b, k, -1), qs)
    want = body(None, 0.0, opt.sparse_embed.embedding[ids].view(b, k, -1), qs)
    torch.testing.assert_close(logit + 0.0, want, rtol=1e-5, atol=1e-6)
    assert opt.looked_up == [] and opt.scored == [(model, (b, k), 0.0, 0.0, reg)]


@pytest.mark.parametrize("body,model,n_q,mul,cen", [(_native_box, "box", 2, 1, 0.02), (_native_vec, "l1", 1, 1, 0.0),
                                                      (_native_rotate, "rotate", 2, 2, 0.0)])
@pytest.mark.parametrize("branches", [1, 2])
@pytest.mark.parametrize("shared", [False, True])
def test_native_cal_logit_bodies_become_one_fused_request(body, model, n_q, mul, cen, branches, shared):
    """The torch-operator form of the logits (--logit_impl native): no lookup, one request with the model, margin
    and coefficient the ext_ops form gives, and the value of the torch expression on the rows."""
    n, d, b, k = 40, 6, 3, 5
    be = 1 if shared else b
    opt = RecordingOptimizer(n, mul * d)
    ids = torch.randint(0, n, (be * k,), generator=torch.Generator().manual_seed(21))
    qs = _queries(b, branches, d, n_q, 22)
    gamma = torch.nn.Parameter(torch.Tensor([12.0]), requires_grad=False)
    logit = body(gamma, cen, LazyRows(opt, ids, "negative_entity").view(be, k, -1), qs)
    want = body(gamma, cen, opt.sparse_embed.embedding[ids].view(be, k, -1), qs)
    torch.testing.assert_close(logit + 0.0, want, rtol=1e-5, atol=1e-6)        # (the first use scores the placeholder)
    assert opt.looked_up == [] and opt.scored == [(model, (be, k), 12.0, cen, None)]


def _native_beta(gamma, entity_embedding, query_embedding):
    """native_cal_logit of models/beta.py:293-301"""
    import torch.distributions.kl as torch_kl
    alpha_embedding, beta_embedding = torch.chunk(entity_embedding.unsqueeze(1), 2, dim=-1)
    entity_dist = ext_ops.BetaDist(alpha_embedding, beta_embedding)
    query_dist = ext_ops.BetaDist(*query_embedding)
    kld = torch_kl._kl_beta_beta(entity_dist, query_dist)
    logit = gamma - torch.norm(kld, p=1, dim=-1)
    return torch.max(logit, dim=1)[0]


@pytest.mark.parametrize("leaf_queries", [True, False])
@pytest.mark.parametrize("branches", [1, 2])
def test_native_beta_body_is_recognised_node_for_node(leaf_queries, branches):
    """torch's own Beta-Beta KL routine on the halves of the regularized handle: one request for beta_kl with the
    clamp prologue; the query-side operands are identified through the autograd graph (leaves, and two outputs of one
    chunk node as the query nets produce them)."""
    n, d, b, k = 40, 5, 3, 4
    opt = RecordingOptimizer(n, 2 * d)
    ids = torch.randint(0, n, (b * k,), generator=torch.Generator().manual_seed(41))
    g = torch.Generator().manual_seed(42)
    if leaf_queries:
        qs = [(torch.rand((b, branches, 1, d), generator=g) + 0.1).requires_grad_(True) for _ in range(2)]
    else:
        both = (torch.rand((b, branches, 1, 2 * d), generator=g) + 0.1).requires_grad_(True)
        qs = list(torch.chunk(both * 1.0, 2, dim=-1))
    gamma = torch.nn.Parameter(torch.Tensor([60.0]), requires_grad=False)
    reg = lambda x: torch.clamp(x + 1.0, 0.05, 1e9)                       # Regularizer(1, 0.05, 1e9), beta.py:210
    logit = _native_beta(gamma, reg(LazyRows(opt, ids, "negative_entity").view(b, k, -1)), qs)
    want = _native_beta(gamma, reg(opt.sparse_embed.embedding[ids].view(b, k, -1)), qs)
    torch.testing.assert_close(logit + 0.0, want.detach(), rtol=1e-5, atol=1e-5)
    assert opt.looked_up == [] and opt.scored == [("beta_kl", (b, k), 60.0, 0.0, (1.0, 0.05, 1e9))]


def test_expressions_that_only_resemble_the_beta_routine_are_evaluated_by_torch():
    """Another tensor in the place of lgamma(qa + qb), queries without a graph, a swapped pair of halves: no request,
    the torch value."""
    import torch.distributions.kl as torch_kl
    n, d, b, k = 40, 5, 3, 4
    ids = torch.randint(0, n, (b * k,), generator=torch.Generator().manual_seed(43))
    g = torch.Generator().manual_seed(44)
    reg = lambda x: torch.clamp(x + 1.0, 0.05, 1e9)
    qa, qb = [(torch.rand((b, 1, 1, d), generator=g) + 0.1).requires_grad_(True) for _ in range(2)]

    def kl_with(p1, p0, q1, q0, y=None):          # torch's routine with its lgamma(sq) replaceable
        sp, sq = p1 + p0, q1 + q0
        t1 = q1.lgamma() + q0.lgamma() + sp.lgamma()
        t2 = p1.lgamma() + p0.lgamma() + (sq.lgamma() if y is None else y)
        return t1 - t2 + (p1 - q1) * torch.digamma(p1) + (p0 - q0) * torch.digamma(p0) + (sq - sp) * torch.digamma(sp)

    cases = {"other tensor": lambda a, c: kl_with(a, c, qa, qb, y=(qa * qb).lgamma()),
             "no graph, other tensor": lambda a, c: kl_with(a, c, qa.detach(), qb.detach(), y=(qa * qb).detach().lgamma()),
             "graph on one side only": lambda a, c: kl_with(a, c, qa, qb.detach()),
             "halves swapped": lambda a, c: kl_with(c, a, qa, qb),
             "queries swapped in one term": lambda a, c: kl_with(a, c, qa, qb) + ((a - qb) * torch.digamma(a) - (a - qa) * torch.digamma(a))}
    for name, f in cases.items():
        opt = RecordingOptimizer(n, 2 * d)
        rows = reg(opt.sparse_embed.embedding[ids].view(b, k, -1)).unsqueeze(1)
        handle = reg(LazyRows(opt, ids, None).view(b, k, -1)).unsqueeze(1)
        got = torch.norm(f(*torch.chunk(handle, 2, dim=-1)), p=1, dim=-1)
        want = torch.norm(f(*torch.chunk(rows, 2, dim=-1)), p=1, dim=-1)
        assert isinstance(got, torch.Tensor) and opt.scored == [], name
        torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-6)
    # and the routine itself on these operands is recognised
    opt = RecordingOptimizer(n, 2 * d)
    handle = reg(LazyRows(opt, ids, None).view(b, k, -1)).unsqueeze(1)
    a, c = torch.chunk(handle, 2, dim=-1)
    kld = torch_kl._kl_beta_beta(ext_ops.BetaDist(a, c), ext_ops.BetaDist(qa, qb))
    assert not isinstance(torch.norm(kld, p=1, dim=-1), torch.Tensor)
    # ... and under no_grad, where the query-side operands are compared by value
    with torch.no_grad():
        a, c = torch.chunk(reg(LazyRows(opt, ids, None).view(b, k, -1)).unsqueeze(1), 2, dim=-1)
        kld = torch_kl._kl_beta_beta(ext_ops.BetaDist(a, c), ext_ops.BetaDist(qa.detach(), qb.detach()))
        assert not isinstance(torch.norm(kld, p=1, dim=-1), torch.Tensor)


@pytest.mark.parametrize("norm", [False, True])
def test_complex_matrix_product_branch_for_shared_negatives(norm):
    """complex.py:178-186: halves of the [1, K] rows viewed as [K, h], transposed, torch.mm with the query matrices,
    added -- one request for the K shared ids; the pieces put to other uses are torch's values."""
    n, d, b, k = 40, 6, 3, 5
    opt = RecordingOptimizer(n, 2 * d)
    ids = torch.randint(0, n, (k,), generator=torch.Generator().manual_seed(51))
    q_re, q_im = _queries(b, 1, d, 2, 52)
    embed_norm = _Normalizer() if norm else (lambda x: x)

    def branch(entity_embedding):
        re, im = torch.chunk(entity_embedding.unsqueeze(1), 2, dim=-1)
        re, im = embed_norm(re), embed_norm(im)
        assert re.shape[0] != q_re.shape[0]
        re, im = re.view(k, d), im.view(k, d)
        return torch.mm(q_re.view(b, d), re.t()) + torch.mm(q_im.view(b, d), im.t())

    logit = branch(LazyRows(opt, ids, "negative_entity").view(1, k, -1))
    want = branch(opt.sparse_embed.embedding[ids].view(1, k, -1))
    assert tuple(logit.shape) == (b, k)
    torch.testing.assert_close(logit + 0.0, want, rtol=1e-5, atol=1e-6)
    assert opt.looked_up == [] and opt.scored == [("complex", (1, k), 0.0, 0.0, "unit_halves" if norm else None)]
    # pieces on their own
    opt2 = RecordingOptimizer(n, 2 * d)
    rows = opt2.sparse_embed.embedding[ids].view(1, 1, k, -1)
    h_re, h_im = torch.chunk(LazyRows(opt2, ids, None).view(1, k, -1).unsqueeze(1), 2, dim=-1)
    t_re, t_im = torch.chunk(rows, 2, dim=-1)
    assert torch.equal(h_re.view(k, d).t() * 1.0, t_re.view(k, d).t())
    assert torch.equal(torch.mm(q_re.view(b, d), h_re.view(k, d).t()) * 1.0, torch.mm(q_re.view(b, d), t_re.view(k, d).t()))
    assert torch.equal(torch.mm(q_re.view(b, d), h_re.view(k, d).t()) + torch.mm(q_im.view(b, d), h_re.view(k, d).t()),
                       torch.mm(q_re.view(b, d), t_re.view(k, d).t()) + torch.mm(q_im.view(b, d), t_re.view(k, d).t()))
    assert torch.equal(h_im.view(k, d) * 1.0, t_im.view(k, d)) and opt2.scored == []


def test_native_intermediates_put_to_other_uses_are_the_tensors_they_stand_for():
    n, d, b, k = 40, 6, 3, 5
    F = torch.nn.functional
    opt = RecordingOptimizer(n, d)
    ids = torch.randint(0, n, (b * k,), generator=torch.Generator().manual_seed(23))
    c, o = _queries(b, 2, d, 2, 24)
    other = _queries(b, 2, d, 1, 25)[0]
    rows = opt.sparse_embed.embedding[ids].view(b, k, -1)
    handle = LazyRows(opt, ids, None).view(b, k, -1)
    delta = (handle.unsqueeze(1) - c).abs()
    t_delta = (rows.unsqueeze(1) - c).abs()
    assert delta.shape == t_delta.shape and opt.looked_up == []
    assert torch.equal(delta * 2.0, t_delta * 2.0)
    assert torch.equal(F.relu(delta - o) + 1.0, F.relu(t_delta - o) + 1.0)
    assert torch.equal(torch.min(delta, o).sum(-1), torch.min(t_delta, o).sum(-1))
    assert torch.equal(torch.norm(F.relu(delta - o), p=2, dim=-1), torch.norm(F.relu(t_delta - o), p=2, dim=-1))
    assert torch.equal(torch.norm(delta, p=1, dim=-1), torch.norm(t_delta, p=1, dim=-1))      # |e - c| has no model
    assert torch.equal((handle.unsqueeze(1) - c).abs() - 0.5, t_delta - 0.5)                  # a scalar is no offset
    assert torch.equal(handle.unsqueeze(1) - c[0, 0, 0], rows.unsqueeze(1) - c[0, 0, 0])      # a 1-D operand is no query
    assert len(opt.looked_up) == 1 and opt.scored == []
    # box_out and box_in with different offsets: two terms that do not share their operands
    logit = 24.0 - torch.norm(F.relu(delta - o), p=1, dim=-1) - 0.02 * torch.norm(torch.min(delta, other), p=1, dim=-1)
    assert logit._fusable() is None


def test_other_uses_fall_back_to_one_lookup():
    n, d, b, k = 30, 4, 2, 3
    opt = RecordingOptimizer(n, d)
    ids = torch.randint(0, n, (b * k,), generator=torch.Generator().manual_seed(7))
    rows = LazyRows(opt, ids, "negative_entity")
    table = opt.sparse_embed.embedding
    assert torch.equal(torch.norm(rows, p=3), torch.norm(table[ids], p=3))             # cal_reg, kg_reasoning.py:149-152
    assert torch.equal(rows.view(b, k, -1)[1], table[ids].view(b, k, -1)[1])            # indexing
    assert torch.equal(rows * 2.0, table[ids] * 2.0) and torch.equal(1.0 - rows, 1.0 - table[ids])
    assert torch.equal(rows.view(b, k, 2, 2), table[ids].view(b, k, 2, 2))              # rows split: values needed
    assert opt.looked_up == ["negative_entity"], "one lookup per handle family"
    assert rows.shape == (b * k, d) and rows.dim() == 2 and rows.size(0) == b * k and len(rows) == b * k


def test_expressions_the_scorer_has_no_model_for_use_the_dense_route():
    """Two different handles in one expression, or a coefficient on box_out, evaluate term by term."""
    n, d, b, k = 30, 4, 2, 3
    opt = RecordingOptimizer(n, d)
    ids = torch.randint(0, n, (b * k,), generator=torch.Generator().manual_seed(8))
    c, o = _queries(b, 1, d, 2, 9)
    rows = LazyRows(opt, ids, None).view(b, k, -1)
    logit = 24.0 - 2.0 * ext_ops.box_dist_out(rows, c, o)
    assert logit._fusable() is None
    other = LazyRows(opt, ids.flip(0), None).view(b, k, -1)
    mixed = 24.0 - ext_ops.box_dist_out(rows, c, o) - 0.02 * ext_ops.box_dist_in(other, c, o)
    assert mixed._fusable() is None
    assert (24.0 - ext_ops.box_dist_out(rows, c, o) - 0.5 * ext_ops.box_dist_in(rows, c, o))._fusable() == ("box", 0.5)
    assert (24.0 - ext_ops.box_dist_out(rows, c, o))._fusable() == ("box", 0.0)


def test_scalar_tensor_values_are_not_confused_between_tensors():
    """The margin's value is cached per tensor object and version; a new tensor never inherits an old entry."""
    n, d = 10, 4
    opt = RecordingOptimizer(n, d)
    rows = LazyRows(opt, torch.arange(4), None).view(2, 2, -1)
    q = _queries(2, 1, d, 1, 10)[0]
    for value in (3.0, 5.0, 7.0):
        gamma = torch.tensor([value])
        assert (gamma - ext_ops.l1_dist(rows, q)).const == value
        del gamma
    gamma = torch.tensor([1.0])
    assert (gamma - ext_ops.l1_dist(rows, q)).const == 1.0
    gamma.fill_(2.0)
    assert (gamma - ext_ops.l1_dist(rows, q)).const == 2.0


def test_positives_and_negatives_of_one_query_batch_share_one_launch():
    """kg_reasoning.py:340-355: positives [B] and negatives [B,K] are scored against the same query tensors by two
    cal_logit calls.  With one union branch both logits stay pending after torch.max; the first use evaluates both
    in one request with the ids side by side, and each gets its own columns."""
    n, d, b, k = 60, 8, 4, 6
    opt = RecordingOptimizer(n, d)
    gen = torch.Generator().manual_seed(2)
    pos, neg = torch.randint(0, n, (b,), generator=gen), torch.randint(0, n, (b, k), generator=gen)
    c, o = _queries(b, 1, d, 2, 12)
    gamma = torch.nn.Parameter(torch.tensor([24.0]), requires_grad=False)

    def cal_logit(rows):
        logit = gamma - ext_ops.box_dist_out(rows, c, o) - 0.02 * ext_ops.box_dist_in(rows, c, o)
        return torch.max(logit, dim=1)[0]

    lp = cal_logit(LazyRows(opt, pos, "positive_entity").unsqueeze(1))
    ln = cal_logit(LazyRows(opt, neg.view(-1), "negative_entity").view(b, k, -1))
    assert not opt.scored and len(opt.pending_scores) == 2 and lp.shape == (b, 1) and ln.shape == (b, k)
    loss = -torch.nn.functional.logsigmoid(lp).mean() - torch.nn.functional.logsigmoid(-ln).mean()
    assert opt.scored == [("box", (b, 1 + k), 24.0, 0.02, None)] and not opt.pending_scores and not opt.looked_up
    table = opt.sparse_embed.embedding
    want_p = (24.0 - _textbook("box", table[pos].unsqueeze(1), (c, o), 0.02))[:, 0]
    want_n = (24.0 - _textbook("box", table[neg], (c, o), 0.02))[:, 0]
    assert torch.allclose(lp.materialize(), want_p, atol=1e-5) and torch.allclose(ln.materialize(), want_n, atol=1e-5)
    want = -torch.nn.functional.logsigmoid(want_p).mean() - torch.nn.functional.logsigmoid(-want_n).mean()
    assert torch.allclose(loss, want, atol=1e-6)
    # other queries, another margin or several branches do not join
    c2, o2 = _queries(b, 1, d, 2, 13)
    other = torch.max(24.0 - ext_ops.box_dist_out(LazyRows(opt, neg.view(-1), None).view(b, k, -1), c2, o2), dim=1)[0]
    again = cal_logit(LazyRows(opt, pos, None).unsqueeze(1))
    assert len(opt.pending_scores) == 2
    float(again.sum())
    assert opt.scored[-1] == ("box", (b, 1), 24.0, 0.02, None) and len(opt.pending_scores) == 1
    values, indices = torch.max(24.0 - ext_ops.l1_dist(LazyRows(opt, pos, None).unsqueeze(1), c), dim=1)
    assert indices.shape == (b, 1) and int(indices.sum()) == 0


def test_shared_negatives_wait_beside_per_query_positives():
    """--share_negative gives negative ids [1,K] (online_sampler.py:155-157) next to positives [B]: both wait for
    the first use, then the per-query ids go into one launch and the shared ids, still K of them, into another
    (never expanded to [B, K])."""
    n, d, b, k = 50, 8, 5, 7
    opt = RecordingOptimizer(n, d)
    gen = torch.Generator().manual_seed(4)
    pos, neg = torch.randint(0, n, (b,), generator=gen), torch.randint(0, n, (1, k), generator=gen)
    (q,) = _queries(b, 1, d, 1, 21)
    cal_logit = lambda rows: torch.max(12.0 - ext_ops.l1_dist(rows, q), dim=1)[0]
    lp = cal_logit(LazyRows(opt, pos, "positive_entity").unsqueeze(1))
    ln = cal_logit(LazyRows(opt, neg.view(-1), "negative_entity").view(1, k, -1))
    assert lp.shape == (b, 1) and ln.shape == (b, k)
    total = lp.sum() + ln.sum()
    assert opt.scored == [("l1", (b, 1), 12.0, 0.0, None), ("l1", (1, k), 12.0, 0.0, None)]
    table = opt.sparse_embed.embedding
    want = (12.0 - _textbook("l1", table[pos].unsqueeze(1), (q,), 0.0)).sum() + \
        (12.0 - _textbook("l1", table[neg].expand(b, k, d), (q,), 0.0)).sum()
    assert torch.allclose(total, want, atol=1e-4)
    alone = cal_logit(LazyRows(opt, neg.view(-1), "negative_entity").view(1, k, -1))
    float(alone.sum())
    assert opt.scored[-1] == ("l1", (1, k), 12.0, 0.0, None)


def test_pending_scores_behave_as_the_tensor_they_stand_for():
    """What training and evaluation code does with the logits (train_process.py:112-128, 194-213): arithmetic from
    both sides, comparison, indexing, iteration, cat / stack / argsort / softmax, views and reductions."""
    n, d, b, k = 60, 8, 4, 6
    opt = RecordingOptimizer(n, d)
    gen = torch.Generator().manual_seed(2)
    pos, neg = torch.randint(0, n, (b,), generator=gen), torch.randint(0, n, (b, k), generator=gen)
    c, o = _queries(b, 1, d, 2, 12)
    cal = lambda rows: torch.max(24.0 - ext_ops.box_dist_out(rows, c, o) - 0.02 * ext_ops.box_dist_in(rows, c, o), dim=1)[0]
    fresh = lambda: (cal(LazyRows(opt, pos, None).unsqueeze(1)), cal(LazyRows(opt, neg.view(-1), None).view(b, k, -1)))
    table = opt.sparse_embed.embedding
    want_p = (24.0 - _textbook("box", table[pos].unsqueeze(1), (c, o), 0.02))[:, 0]
    want_n = (24.0 - _textbook("box", table[neg], (c, o), 0.02))[:, 0]
    uses = [
        lambda lp, ln: (torch.cat([lp, ln], dim=1), torch.cat([want_p, want_n], dim=1)),
        lambda lp, ln: (torch.stack([ln, ln]), torch.stack([want_n, want_n])),
        lambda lp, ln: (torch.nn.functional.logsigmoid(lp).squeeze(dim=1), torch.nn.functional.logsigmoid(want_p).squeeze(dim=1)),
        lambda lp, ln: ((ln > 20).sum(), (want_n > 20).sum()),
        lambda lp, ln: (torch.argsort(ln, dim=1, descending=True), torch.argsort(want_n, dim=1, descending=True)),
        lambda lp, ln: (ln[1], want_n[1]),
        lambda lp, ln: (torch.stack(list(ln)), want_n),
        lambda lp, ln: (torch.softmax(ln * 0.5, dim=1).detach() * torch.nn.functional.logsigmoid(-ln),
                        torch.softmax(want_n * 0.5, dim=1) * torch.nn.functional.logsigmoid(-want_n)),
        lambda lp, ln: (torch.ones(b, k) * ln + (1.0 - ln) / 2, want_n + (1.0 - want_n) / 2),
        lambda lp, ln: (ln.view(-1), want_n.reshape(-1)),
        lambda lp, ln: (ln.t().sum(dim=0) + lp.mean(), want_n.sum(dim=1) + want_p.mean()),
    ]
    for use in uses:
        got, want = use(*fresh())
        assert got.shape == want.shape and torch.allclose(got.float(), want.float(), atol=1e-4)
    lp, ln = fresh()
    assert len(ln) == b and ln.size(1) == k and ln.dim() == 2 and ln.numel() == b * k and ln.dtype == torch.float32
    assert abs(float(lp.sum()) - float(want_p.sum())) < 1e-3


def test_a_placeholder_nobody_holds_is_never_scored():
    """An evaluation loop that ignores one of the two logits (train_process.py:112-128 takes the negative ones only)
    must not leave work or memory behind: the optimizer holds pending scores by weak reference."""
    import gc
    n, d, b, k = 40, 8, 3, 5
    opt = RecordingOptimizer(n, d)
    (q,) = _queries(b, 1, d, 1, 31)
    ids = torch.randint(0, n, (b, k), generator=torch.Generator().manual_seed(6))
    cal = lambda rows: torch.max(12.0 - ext_ops.l1_dist(rows, q), dim=1)[0]
    for _ in range(3):
        dropped = cal(LazyRows(opt, ids[:, 0], None).unsqueeze(1))
        del dropped
    gc.collect()
    kept = cal(LazyRows(opt, ids.view(-1), None).view(b, k, -1))
    float(kept.sum())
    assert opt.scored == [("l1", (b, k), 12.0, 0.0, None)] and not opt.pending_scores


def test_handles_leave_no_reference_cycles():
    """A handle family can hold gigabytes (the ids, the looked-up rows): everything must go when the model code
    lets go of it, by reference count, not at some later pass of the cycle collector."""
    import gc
    n, d, b, k = 60, 8, 4, 6
    opt = RecordingOptimizer(n, d)
    c, o = _queries(b, 1, d, 2, 12)
    ids = torch.randint(0, n, (b, k), generator=torch.Generator().manual_seed(3))

    def fused_use():
        rows = LazyRows(opt, ids.view(-1), None)
        rows.job_handle.sync()
        rows = rows.view(b, k, -1)
        values, which = torch.max(24.0 - ext_ops.box_dist_out(rows, c, o) - 0.02 * ext_ops.box_dist_in(rows, c, o), dim=1)
        return float(values.sum()) + float(which.sum())

    def plain_use():
        rows = LazyRows(opt, ids.view(-1), None).view(b, k, -1)
        return float(torch.norm(rows + 1.0, p=3))

    gc.collect()
    gc.disable()
    try:
        for use in (fused_use, plain_use):
            use()
            assert gc.collect() == 0, use.__name__
    finally:
        gc.enable()


def test_a_handle_on_the_query_side_is_looked_up():
    """The reverse layout of inverse queries hands the negatives to the operator as the QUERY operand
    (kg_reasoning.py:257-263): a handle there has nothing to fuse and stands for its rows."""
    n, d, b, k = 30, 8, 3, 4
    opt = RecordingOptimizer(n, d)
    gen = torch.Generator().manual_seed(8)
    tail, neg = torch.randint(0, n, (b,), generator=gen), torch.randint(0, n, (b, k), generator=gen)
    table = opt.sparse_embed.embedding
    entity = table[tail].unsqueeze(1).contiguous()                                   # [B,1,D] tensor
    queries = LazyRows(opt, neg.view(-1), "negative_entity").view(b, k, -1)         # [B,K,D] handle
    want = _textbook("l1", entity, (table[neg],), 0.0)
    try:
        got = ext_ops.l1_dist(entity, queries)
    except Exception as e:                                                          # no GPU here: the dense operator needs the library's kernels
        assert "materialize" not in str(e) and "LazyRows" not in str(e), e
        assert opt.looked_up == ["negative_entity"]
        return
    assert torch.allclose(got, want, atol=1e-5)


def test_comparisons_and_the_rarer_operators_give_what_the_tensor_gives():
    """`rows == 0`, `logit != x` with a Python scalar must be elementwise tensors, not object identity; the
    operators a handle has no lazy form for (%, **, &, item assignment) compute on the rows it stands for."""
    n, d, b, k = 20, 4, 2, 3
    opt = RecordingOptimizer(n, d)
    ids = torch.randint(0, n, (b * k,), generator=torch.Generator().manual_seed(11))
    rows = LazyRows(opt, ids, "negative_entity")
    table = opt.sparse_embed.embedding
    want = table[ids]
    assert torch.equal(rows == 0, want == 0) and torch.equal(rows != 0.25, want != 0.25)
    assert torch.equal(0.0 == rows, want == 0.0) and torch.equal(rows == want, torch.ones_like(want, dtype=torch.bool))
    assert torch.equal(rows % 0.3, want % 0.3) and torch.equal(2.0 ** rows, 2.0 ** want)
    assert torch.equal(rows // 0.3, want // 0.3) and torch.equal(+rows, want)
    assert torch.equal((rows > 0) & (rows < 1), (want > 0) & (want < 1))
    assert torch.equal((rows > 0) | (rows < -1), (want > 0) | (want < -1))
    assert isinstance(hash(rows), int) and len({rows: 1}) == 1        # still usable as a dictionary key
    (c,) = _queries(b, 1, d, 1, 12)
    logit = 12.0 - ext_ops.l1_dist(LazyRows(opt, ids, None).view(b, k, -1), c)
    value = logit.materialize()
    assert torch.equal(logit == value, torch.ones_like(value, dtype=torch.bool))
    assert torch.equal(logit != 12.0, value != 12.0)
    copy = LazyRows(opt, ids, None)
    copy[0] = 0.0                                                       # writes into the looked-up rows
    assert float(copy.materialize()[0].abs().sum()) == 0.0
