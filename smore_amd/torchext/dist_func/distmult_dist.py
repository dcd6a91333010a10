"""DistMult similarity (surface of smore/common/torchext/dist_func/distmult_dist.py)."""
from ._base import apply_dist


def distmult_sim(entity_embed, center_embed):
    return apply_dist("distmult", entity_embed, center_embed)


def naive_innerprod(entity_embedding, query_embedding):
    return (entity_embedding * query_embedding).sum(dim=-1)
