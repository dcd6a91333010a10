"""Shared machinery of the distance operators.

One autograd Function serves every operator kind; the public modules next to
this file (l1_dist.py, box_dist.py, ...) only bind names.  Behaviour follows
the per-operator Functions of smore/common/torchext/dist_func/*.py:
  * inputs must be contiguous 3-D tensors whose leading two extents divide one
    another pairwise; a violated precondition is an AssertionError, as there
    (l2_dist.py:25-29, rotate_dist.py:25-31);
  * the result is [max(be,bc), max(ne,nc)] (l2_dist.py:31-32);
  * backward returns one gradient per tensor input, shaped like the input
    (l2_dist.py:38-45);
  * a 4-D query [bc, U, nc, D] is scored branch by branch along dim 1 and the
    results stacked on dim 1 (box_dist.py:50-61).
"""
import torch

from ... import extlib_hip as extlib
from ...embedding.lazy_rows import LazyRows, _is_lazy, lazy_dist

TWO_HALVES = ("rotate", "complex", "beta_kl", "beta_l2", "beta_fisher_approx")


class DistFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, kind, entity_embed, *queries):
        first = queries[0]
        mul = 2 if kind in TWO_HALVES else 1
        for t in (entity_embed,) + queries:
            assert t.dim() == 3
            assert t.is_contiguous()
        assert entity_embed.shape[-1] == first.shape[-1] * mul
        for q in queries[1:]:
            assert q.shape == first.shape
        assert entity_embed.shape[0] % first.shape[0] == 0 or first.shape[0] % entity_embed.shape[0] == 0
        assert entity_embed.shape[1] % first.shape[1] == 0 or first.shape[1] % entity_embed.shape[1] == 0
        rows = max(entity_embed.shape[0], first.shape[0])
        cols = max(entity_embed.shape[1], first.shape[1])
        with torch.no_grad():
            dst = entity_embed.new_empty((rows, cols))
            second = queries[1] if len(queries) == 2 else None
            extlib.dist_forward(kind, entity_embed, first, second, dst, second is not None)
        ctx.kind = kind
        ctx.save_for_backward(entity_embed.detach(), *[q.detach() for q in queries])
        return dst

    @staticmethod
    def backward(ctx, grad_out):
        entity_embed, *queries = ctx.saved_tensors
        with torch.no_grad():
            grad_out = grad_out.contiguous()
            grads = [torch.empty_like(t) for t in (entity_embed, *queries)]  # kernels overwrite every element
            second = queries[1] if len(queries) == 2 else None
            gsecond = grads[2] if len(queries) == 2 else None
            extlib.dist_backward(ctx.kind, grad_out, entity_embed, queries[0], second, grads[0], grads[1], gsecond,
                                 second is not None)
        return (None, *grads)


def apply_dist(kind, entity_embed, *queries):
    """3-D or (query) 4-D front end shared by every operator.  An entity argument that is a lazy lookup handle
    (what sp_embed(ids) returns while an EmbeddingOptimizer is attached) gives a lazy distance: the table rows are
    then read by the gather-fused scorer when the logit is needed, never as a [B,K,row] tensor."""
    if isinstance(entity_embed, LazyRows):
        lazy = lazy_dist(kind, entity_embed, *queries) if kind != "l2" else None   # "l2" here is the squared distance
        if lazy is not None:
            return lazy
        entity_embed = entity_embed.materialize().contiguous()
    # a lookup handle (or a pending score) on the query side has nothing to fuse: the operator gets its values
    queries = [q.materialize() if _is_lazy(q) else q for q in queries]
    first = queries[0]
    if entity_embed.dim() != first.dim():
        assert first.dim() == 4
        assert entity_embed.dim() == 3
        per_branch = []
        for u in range(first.shape[1]):
            branch = [q[:, u, :, :].contiguous() for q in queries]
            per_branch.append(DistFunction.apply(kind, entity_embed, *branch))
        return torch.stack(per_branch, dim=1)
    assert entity_embed.dim() == 3 and all(q.dim() == 3 for q in queries)
    return DistFunction.apply(kind, entity_embed, *queries)
