"""L2 distance operator (surface of smore/common/torchext/dist_func/l2_dist.py:21-62).

The native operator returns the squared distance; the square root is taken
here, outside the Function, so autograd supplies g / (2 sqrt(d2)) -- infinite
at d2 == 0, exactly as in the reference (l2_dist.py:59,62)."""
import torch

from ...embedding.lazy_rows import LazyRows, lazy_dist
from ._base import apply_dist


def l2_sqr_dist(entity_embed, center_embed):
    return apply_dist("l2", entity_embed, center_embed)


def l2_dist(entity_embed, center_embed):
    if isinstance(entity_embed, LazyRows):     # a lazy lookup: the fused scorer has the rooted distance as a model
        lazy = lazy_dist("l2", entity_embed, center_embed)
        if lazy is not None:
            return lazy
    return torch.sqrt(l2_sqr_dist(entity_embed, center_embed))


def naive_l2(entity_embedding, query_embedding):
    """Pure-torch twin (l2_dist.py:65-67)."""
    return torch.norm(entity_embedding - query_embedding, p=2, dim=-1)
