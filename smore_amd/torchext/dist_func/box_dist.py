"""Query2box distances (surface of smore/common/torchext/dist_func/box_dist.py:21-76)."""
import torch
import torch.nn.functional as F

from ._base import apply_dist


def box_dist(entity_embed, center_embed, offset_embed, dist_type):
    assert dist_type in ("in", "out")
    return apply_dist("box_" + dist_type, entity_embed, center_embed, offset_embed)


def box_dist_out(entity_embed, center_embed, offset_embed):
    return box_dist(entity_embed, center_embed, offset_embed, "out")


def box_dist_in(entity_embed, center_embed, offset_embed):
    return box_dist(entity_embed, center_embed, offset_embed, "in")


def naive_box_dist_out(entity_embedding, query_center_embedding, query_offset_embedding):
    """Pure-torch twin (box_dist.py:78-82)."""
    delta = (entity_embedding - query_center_embedding).abs()
    return torch.norm(F.relu(delta - query_offset_embedding), p=1, dim=-1)


def naive_box_dist_in(entity_embedding, query_center_embedding, query_offset_embedding):
    """Pure-torch twin (box_dist.py:85-89)."""
    delta = (entity_embedding - query_center_embedding).abs()
    return torch.norm(torch.min(delta, query_offset_embedding), p=1, dim=-1)
