"""Entity table kept in HBM, with the calling surface of smore/common/embedding/sparse_embed.py:26-67.

Model code of the reference talks to the table through three things only: `entity_embedding(ids, name)`
returns rows carrying a `.job_handle` whose `.sync()` it may call, `entity_embedding(None)` returns the
whole table (evaluation against all entities), and an `EmbeddingOptimizer` may install itself as
`fwd_delegate` to take the lookups over (embed_optimizer.py:116-121).  This class keeps exactly that
contract; the rows themselves come from the HIP gather, and the optimizer state the optimizers register
(`register_tensor`) becomes part of the module's state_dict under the reference's buffer names.
"""
import torch
from torch import nn

from .. import _lib, fused


class DummyJob:
    """Handle of a lookup that is already complete (the role of embed_rw.py's DummyJob): rows gathered
    on the device are ordered by the stream, so there is nothing for the caller to wait for."""

    __slots__ = ()

    def sync(self):
        return None


_DONE = DummyJob()


class SparseEmbedding(nn.Module):
    """[num_rows, num_cols] fp32 table whose rows are read by id and updated sparsely.

    Attributes used by callers: `embedding` (the nn.Parameter), `num_rows`, `fwd_delegate`, `dummy_job`,
    `device`, `shape`."""

    def __init__(self, num_rows, num_cols):
        super().__init__()
        if num_rows < 0 or num_cols <= 0:
            raise ValueError(f"bad table shape {num_rows} x {num_cols}")
        self.num_rows = int(num_rows)
        self.dummy_job = _DONE
        self.fwd_delegate = None  # set by EmbeddingOptimizer.__init__
        self.embedding = nn.Parameter(torch.zeros((self.num_rows, int(num_cols)), dtype=torch.float32))

    # ---- what callers ask about the table
    shape = property(lambda self: self.embedding.shape)
    device = property(lambda self: self.embedding.device)

    def extra_repr(self):
        return f"rows={self.num_rows}, cols={self.embedding.shape[1]}, device={self.embedding.device}"

    # ---- set-up
    def init_params(self, lb, ub):
        """Uniform initial values in [lb, ub) (the reference's embedding_range)."""
        with torch.no_grad():
            self.embedding.uniform_(lb, ub)

    def register_tensor(self, name, tensor_obj):
        """Optimizer state that must be saved and moved with the table (e.g. state_sum_fo / state_sum_sq)."""
        if tensor_obj.shape[0] != self.num_rows:
            raise _lib.SmxError(f"{name}: one state row per table row is needed")
        self.register_buffer(name, tensor_obj)

    # ---- lookups
    def _rows(self, indices):
        table = self.embedding.detach()
        with torch.no_grad():
            return fused.gather_rows(table, indices.to(table.device))

    def forward(self, indices, name=None):
        """Rows `indices` of the table (`None`: the table itself), tagged with a finished job handle.
        With an optimizer attached the lookup is the optimizer's (it records what to update)."""
        if not self.num_rows:
            return None
        delegate = self.fwd_delegate
        if delegate is not None:
            return delegate(indices, name)
        out = self.embedding if indices is None else self._rows(indices)
        out.job_handle = self.dummy_job
        return out
