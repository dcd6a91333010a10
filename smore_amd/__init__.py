"""smore_amd: MI355X (gfx950) implementation of SMORE's negative-sample scoring path.

Sub-modules mirror the reference package layout for this path only:
  smore_amd.extlib_hip            the `extlib_cuda` function set (dense operators)
  smore_amd.torchext.ext_ops      l1_dist, l2_dist, box_dist_in/out, rotate_dist, beta_kl, ...
  smore_amd.embedding             SparseEmbedding and the sparse row optimizers
  smore_amd.fused                 gather-fused scoring + segmented entity gradient + Adam
All arithmetic runs in libsmore_amd.so (hand-written HIP, C ABI in include/smore_amd.h).
"""

__version__ = "0.1.0"
