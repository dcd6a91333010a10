"""L1 distance operator (surface of smore/common/torchext/dist_func/l1_dist.py:21-62)."""
import torch

from ._base import apply_dist


def l1_dist(entity_embed, center_embed):
    return apply_dist("l1", entity_embed, center_embed)


def naive_l1(entity_embedding, query_embedding):
    """Pure-torch twin (l1_dist.py:65-67)."""
    return torch.norm(entity_embedding - query_embedding, p=1, dim=-1)
