"""BetaE distances (surface of smore/common/torchext/dist_func/beta_dist.py:21-80)."""
from collections import namedtuple

import torch

from ._base import apply_dist

BetaDist = namedtuple("BetaDist", ["concentration1", "concentration0"])


def beta_dist(entity_embed, query_dist, dist_name):
    assert dist_name in ("kl", "l2", "fisher_approx")
    return apply_dist("beta_" + dist_name, entity_embed, query_dist.concentration1, query_dist.concentration0)


def beta_kl(entity_embed, query_dist):
    return beta_dist(entity_embed, query_dist, "kl")


def beta_l2(entity_embed, query_dist):
    return beta_dist(entity_embed, query_dist, "l2")


def beta_fisher_approx(entity_embed, query_dist):
    return beta_dist(entity_embed, query_dist, "fisher_approx")


def naive_beta_kl(entity_embedding, query_dist):
    """Pure-torch twin (beta_dist.py:82-86)."""
    alpha, beta = torch.chunk(entity_embedding, 2, dim=-1)
    kld = torch.distributions.kl._kl_beta_beta(BetaDist(alpha, beta), query_dist)
    return torch.norm(kld, p=1, dim=-1)
