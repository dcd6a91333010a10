"""Sparse entity table (surface of smore/common/embedding/sparse_embed.py:26-67).

The table and, once an optimizer is attached, its moment buffers live in HBM for the whole run; row
lookups go through `fwd_delegate` when an EmbeddingOptimizer has installed itself, exactly like the
reference, so model code keeps calling `entity_embedding(ids, name)`.
"""
import torch
import torch.nn as nn

from .. import fused


class DummyJob:
    """Completed-job handle: the in-HBM lookup has nothing to wait for (embed_rw.py DummyJob)."""

    def sync(self):
        return None


class SparseEmbedding(nn.Module):

    def __init__(self, num_rows, num_cols):
        super().__init__()
        self.num_rows = num_rows
        self.embedding = nn.Parameter(torch.zeros(num_rows, num_cols))
        self.fwd_delegate = None
        self.dummy_job = DummyJob()

    @property
    def device(self):
        return self.embedding.device

    @property
    def shape(self):
        return self.embedding.shape

    def init_params(self, lb, ub):
        nn.init.uniform_(tensor=self.embedding, a=lb, b=ub)

    def register_tensor(self, name, tensor_obj):
        self.register_buffer(name, tensor_obj)

    def forward(self, indices, name=None):
        if self.num_rows == 0:
            return None
        if self.fwd_delegate is not None:
            return self.fwd_delegate(indices, name)
        if indices is None:
            mat = self.embedding
        else:
            with torch.no_grad():
                mat = fused.gather_rows(self.embedding.detach(), indices.to(self.embedding.device))
        mat.job_handle = self.dummy_job
        return mat
