"""ComplEx similarity (surface of smore/common/torchext/dist_func/complex_dist.py)."""
import torch

from ._base import apply_dist


def complex_sim(entity_embed, re_embed, im_embed):
    return apply_dist("complex", entity_embed, re_embed, im_embed)


def naive_complex_sim(entity_embedding, query_re_embedding, query_im_embedding):
    ent_re, ent_im = torch.chunk(entity_embedding, 2, dim=-1)
    return (ent_re * query_re_embedding + ent_im * query_im_embedding).sum(dim=-1)
