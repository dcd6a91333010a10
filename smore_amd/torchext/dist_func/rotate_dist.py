"""RotatE complex-modulus distance (surface of smore/common/torchext/dist_func/rotate_dist.py:21-65)."""
import torch

from ._base import apply_dist


def rotate_dist(entity_embed, re_embed, im_embed):
    return apply_dist("rotate", entity_embed, re_embed, im_embed)


def naive_rotate_dist(entity_embedding, query_re_embedding, query_im_embedding):
    """Pure-torch twin (rotate_dist.py:68-75)."""
    ent_re, ent_im = torch.chunk(entity_embedding, 2, dim=-1)
    diff = torch.stack([ent_re - query_re_embedding, ent_im - query_im_embedding], dim=0)
    return diff.norm(dim=0).sum(dim=-1)
