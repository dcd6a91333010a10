"""Operator names as imported by the model code (smore/common/torchext/ext_ops.py:15-22)."""
from .dist_func.beta_dist import BetaDist, beta_fisher_approx, beta_kl, beta_l2  # noqa: F401
from .dist_func.box_dist import box_dist_in, box_dist_out  # noqa: F401
from .dist_func.complex_dist import complex_sim  # noqa: F401
from .dist_func.distmult_dist import distmult_sim  # noqa: F401
from .dist_func.l1_dist import l1_dist  # noqa: F401
from .dist_func.l2_dist import l2_dist  # noqa: F401
from .dist_func.rotate_dist import rotate_dist  # noqa: F401
