"""Sparse row optimizer for the entity table (surface of smore/common/embedding/embed_optimizer.py).

Same driver protocol as the reference (training/train_process.py:172-220):
    opt.zero_grad(); rows = sp_embed(ids, name) ... loss.backward(); opt.apply_grad(lr)
and one addition, the gather-fused scorer
    logit = opt.score_negatives(model, ids[B,K], q1, q2, gamma, cen)
which stands for  gamma - dist(regularizer(sp_embed(ids).view(B,K,-1)), query)  without ever
building the [B,K,row] tensor.  Everything after loss.backward() -- unique-merge of ids
(embed_optimizer.py:39-42), segment sum of gradient rows (:45-48) and the lazy Adam update
(:208-252) -- runs as the segment plan and the fused entity pass of libsmore_amd.so.
"""
import warnings
from abc import ABC, abstractmethod

import torch
import torch.nn as nn

from .. import _lib, fused
from .lazy_rows import UNIT_HALVES, UNIT_ROW, LazyRows

_REG_MODEL = {UNIT_HALVES: "complex", UNIT_ROW: "distmult"}     # the one model each unit-length marker belongs to
from .sparse_embed import SparseEmbedding


def merge_grad_indices(idx_list, n_rows):
    """torch.unique(cat(idx_list), return_inverse=True) on the device (embed_optimizer.py:39-42).
    Returns (merged_indices, inverse_indices, plan)."""
    flat = torch.cat([i.reshape(-1) for i in idx_list], dim=0)
    plan = fused.build_plan(flat, n_rows, want_inverse=True)
    return plan.uniq, plan.inverse, plan


def merge_grad_list(grad_list, plan):
    """Segment sum of the concatenated gradient rows (embed_optimizer.py:45-48, reduce='sum')."""
    grads = torch.cat(grad_list, dim=0).contiguous()
    merged = torch.empty((plan.n_uniq, grads.shape[1]), dtype=torch.float32, device=grads.device)
    fused.rows_backward(plan, grads, merged=merged)
    return merged


class EmbedLookupFunc(torch.autograd.Function):
    """rows = table[indices]; backward hands (indices, grad_rows) to the optimizer
    (embed_optimizer.py:51-66)."""

    @staticmethod
    def forward(ctx, embed_opt, dummy_tensor, indices, name):
        ctx.embed_opt = embed_opt
        ctx.indices = indices
        ctx.idx_fwd = embed_opt.n_fwd
        embed_opt.n_fwd += 1
        with torch.no_grad():
            table = embed_opt.sparse_embed.embedding.detach()
            return fused.gather_rows(table, indices.to(table.device), embed_opt.err_flag)

    @staticmethod
    def backward(ctx, grad_output):
        ctx.embed_opt.accumulate_grad(ctx.indices, grad_output, ctx.idx_fwd)
        return None, None, None, None


class _FusedScoreFunc(torch.autograd.Function):
    """logit[b,k] = gamma - dist(table[ids[b,k]], q[b]); the entity gradient is not returned to
    autograd but recorded with the optimizer, which reduces it per entity in apply_grad."""

    @staticmethod
    def forward(ctx, embed_opt, dummy_tensor, model, ids, params, q1, q2, for_training=True, branches=1):
        """q1 / q2 [B * branches, dim].  ids [1, K] against more than one query row: negatives shared by the batch
        (--share_negative), they stay K ids and every row scores them: returns [B * branches, K].  Else ids [B, K];
        with branches > 1 (union queries) the result is the maximum over a query's branch rows, [B, K], and the
        second output says which branch held it ([B, K] int64; empty for one branch)."""
        table = embed_opt.sparse_embed.embedding.detach()
        ctx.shared = ids.shape[0] == 1 and q1.shape[0] > 1
        ctx.branches = 1 if ctx.shared else branches
        ctx.winner = None
        with torch.no_grad():
            if ctx.shared:
                codes = None
                score = fused.score_forward_shared(model, table, ids.reshape(-1), q1, q2, params, embed_opt.err_flag)
            elif branches > 1:
                codes = None
                score, ctx.winner = fused.score_forward_union(model, table, ids, q1, q2, params, branches, embed_opt.err_flag)
            else:
                # box, l1: the forward leaves 2-bit sign codes from which both backward passes work (None otherwise;
                # none either when no backward will follow, e.g. scoring sampled negatives under torch.no_grad())
                codes = fused.new_codes(model, table, ids, q1) if for_training and table.shape[1] % 4 == 0 else None
                score = fused.score_forward(model, table, ids, q1, q2, params, embed_opt.err_flag, codes=codes)
        ctx.embed_opt, ctx.model, ctx.ids, ctx.params, ctx.codes = embed_opt, model, ids, params, codes
        ctx.save_for_backward(q1.detach(), q2.detach() if q2 is not None else None, score)
        ctx.idx_fwd = embed_opt.n_fwd
        embed_opt.n_fwd += 1
        index = ctx.winner.long() if ctx.winner is not None else torch.empty(0, dtype=torch.int64, device=score.device)
        ctx.mark_non_differentiable(index)
        return score, index

    @staticmethod
    def backward(ctx, gscore, _gindex):
        q1, q2, score = ctx.saved_tensors
        opt = ctx.embed_opt
        table = opt.sparse_embed.embedding.detach()
        with torch.no_grad():
            gscore = gscore.contiguous()
            if ctx.shared:
                gq1, gq2 = fused.score_backward_query_shared(ctx.model, table, ctx.ids.reshape(-1), q1, q2, score,
                                                             gscore, ctx.params)
            elif ctx.winner is not None:
                gq1, gq2 = fused.score_backward_query_union(ctx.model, table, ctx.ids, q1, q2, score, gscore, ctx.winner,
                                                            ctx.params, ctx.branches)
            else:
                gq1, gq2 = fused.score_backward_query(ctx.model, table, ctx.ids, q1, q2, score, gscore, ctx.params,
                                                      codes=ctx.codes)
        opt.accumulate_fused(ctx.model, ctx.ids, q1, q2, score, gscore, ctx.params, ctx.idx_fwd, ctx.codes,
                             shared=ctx.shared, winner=ctx.winner, branches=ctx.branches)
        return None, None, None, None, None, gq1, gq2, None, None


class EmbeddingOptimizer(ABC):
    """Base driver (embed_optimizer.py:69-163).  `args` needs .optim_mode, a tuple or tuple string
    (mode, name, device, squeeze, queue) as in the reference, and .share_optim_stats."""

    def __init__(self, args, sp_embed, gpu_id=0):
        assert isinstance(sp_embed, SparseEmbedding)
        self.args = args
        self.sparse_embed = sp_embed
        sp_embed.fwd_delegate = self.forward
        self.dummy_tensor = nn.Parameter(torch.randn(1, 1))
        self.grad_list, self.fused_list, self.has_grad_list = [], [], []
        self.pending_scores = []    # weak references to the LazyScores of this step that nothing has needed yet
        self.n_fwd = 0
        self.step = 0
        self.gpu_id = gpu_id
        mode = args.optim_mode
        if isinstance(mode, str):
            mode = tuple(x.strip() for x in mode.strip("()").split(","))
        self.optim_mode = mode
        self.optimizer_name = mode[1]
        # mode[2] is where the reference keeps the optimizer statistics ('gpu' or 'cpu'); here they always live in
        # HBM beside the table, so 'cpu' (what the reference's Freebase scripts pass) is accepted and means the same
        self.optimizer_device = str(mode[2]).strip("'\" ") if len(mode) > 2 else "gpu"
        if self.optimizer_device not in ("gpu", "cpu"):
            raise _lib.SmxError(f"optimizer device must be 'gpu' or 'cpu', got {self.optimizer_device!r}")
        self.squeeze = str(mode[3]).lower() in ("true", "1") if len(mode) > 3 else False
        self.share_optim_stats = getattr(args, "share_optim_stats", True)
        if sp_embed.embedding.device.type != "cuda":
            raise _lib.SmxError("the entity table must live on the GPU (no CPU-table mode in this build)")
        self.err_flag = fused.new_error_flag(sp_embed.embedding.device)
        self.check_ids_every_step = True
        self.check_ids_synchronously = False   # True: every apply_grad waits for the device and raises for its own step
        self._flag_host = torch.zeros(1, dtype=torch.int32, pin_memory=True)   # where the flag of a step lands
        self._flag_event = None                                                # set while such a copy is under way
        self.lazy_lookup = True
        self.stats = self._new_stats()
        self._warned_fallback = False
        # saving the table (state_dict of the SparseEmbedding) is one of the moments a pending id error must surface
        sp_embed.register_state_dict_pre_hook(lambda module, prefix, keep_vars: self.poll_pending_id_check())
        self.prepare_state()

    # -- set-up protocol of the trainer (embed_optimizer.py:71-75, 102-110; called as
    #    get_optim_class(args).prepare_optimizers(args, sparse_embeds) before the workers start)
    @classmethod
    def prepare_embed(cls, args, optim_mode, embed, fn_register):
        """Registers this optimizer's state tensors for `embed` through fn_register(name, tensor)."""

    @classmethod
    def prepare_optimizers(cls, args, list_sparse_embeds):
        if not getattr(args, "share_optim_stats", True):
            return
        mode = args.optim_mode
        if isinstance(mode, str):
            mode = tuple(x.strip() for x in mode.strip("()").split(","))
        for e in list_sparse_embeds:
            assert isinstance(e, SparseEmbedding)
            cls.prepare_embed(args, mode, e, e.register_tensor)

    # -- hooks of the concrete optimizer
    @abstractmethod
    def prepare_state(self):
        ...

    @abstractmethod
    def update_from_plan(self, plan, grad_rows, lr):
        """Segment-sum grad_rows [P,row] over plan and update the table rows of plan.uniq."""

    @abstractmethod
    def update_fused(self, plan, rec, lr):
        """Same for one fused record whose entity gradient is recomputed on the fly."""

    @abstractmethod
    def update_shared(self, plan, rec, lr):
        """Same for one fused record whose K ids are shared by all its queries; plan covers those K ids."""

    @abstractmethod
    def update_fused_multi(self, plan, recs, lr, grad_rows=None):
        """Same for several fused records of one query batch; plan covers their ids in the order of recs, then
        the ids of grad_rows (gradient rows of the step's plain lookups), when there are any."""

    # -- what happened since zero_grad(): how the step's lookups were served
    @staticmethod
    def _new_stats():
        """fused_launches: launches of the gather-fused scorer.  materialized_lookups: plain lookups made for a lazy
        handle (anchors and other uses of the rows themselves; also every fallback).  dense_fallbacks: logits of a
        handle that were evaluated by lookup + dense operators because the fused scorer has no form for them.
        per_record_merges: fused records that apply_grad had to reduce to gradient rows one by one."""
        return dict(fused_launches=0, materialized_lookups=0, dense_fallbacks=0, per_record_merges=0)

    def note_dense_fallback(self, what):
        """Called by the lazy handle when a logit leaves the fused path; says so once per optimizer."""
        self.stats["dense_fallbacks"] += 1
        if not self._warned_fallback:
            self._warned_fallback = True
            warnings.warn(f"smore_amd: {what} is evaluated by plain lookup + dense operators, not by the gather-fused "
                          "scorer (correct results, several times the memory traffic); EmbeddingOptimizer.stats counts "
                          "such steps", RuntimeWarning, stacklevel=3)

    # -- protocol of the training loop
    def zero_grad(self):
        self.poll_pending_id_check(wait=False)   # (never waits for the device: the next step must be free to run ahead)
        self.grad_list, self.fused_list, self.has_grad_list = [], [], []
        self.pending_scores = []
        self.n_fwd = 0
        self.stats = self._new_stats()

    def share_memory(self):
        pass  # state is device memory of one process

    def accumulate_grad(self, indices, grad_submat, fwd_idx):
        self.grad_list.append((indices, grad_submat))
        self.has_grad_list.append(fwd_idx)

    def accumulate_fused(self, model, ids, q1, q2, score, gscore, params, fwd_idx, codes=None, shared=False,
                         winner=None, branches=1):
        self.fused_list.append(dict(model=model, ids=ids, q1=q1, q2=q2, score=score, gscore=gscore, params=params,
                                    codes=codes, fwd_idx=fwd_idx, shared=shared, winner=winner, branches=branches))
        self.has_grad_list.append(fwd_idx)

    def forward(self, indices, name=None):
        """What sp_embed(indices, name) returns while this optimizer is attached (embed_optimizer.py:150-153).
        With lazy_lookup (default) that is a LazyRows handle: model code that only views it, regularizes it and
        hands it to the distance operators of ext_ops gets the gather-fused scorer without knowing; any other use
        turns it into the looked-up rows.  lazy_lookup = False: the rows at once, as in the reference."""
        if indices is None:
            mat = self.sparse_embed.embedding
            mat.job_handle = self.sparse_embed.dummy_job
            return mat
        if self.lazy_lookup:
            return LazyRows(self, indices, name)
        return self.lookup_rows(indices, name)

    def lookup_rows(self, indices, name=None, for_handle=False):
        """rows = table[indices], shaped indices.shape + (row,), through the autograd node that records the
        gradient rows for apply_grad (EmbedLookupFunc, embed_optimizer.py:51-66)."""
        if for_handle:
            self.stats["materialized_lookups"] += 1
        mat = EmbedLookupFunc.apply(self, self.dummy_tensor, indices, name)
        if indices.dim() != 1:
            mat = mat.view(tuple(indices.shape) + (mat.shape[-1],))
        mat.job_handle = self.sparse_embed.dummy_job
        return mat

    def lazy_request(self, model, rows, queries, gamma, cen):
        """What one launch of the fused scorer needs for gamma - dist(rows, queries) with a LazyRows handle
        [Be, K, row] against query tensors [B, 1, D] or [B, U, 1, D]: a dict, or None when this is not a layout the
        fused scorer takes."""
        q = queries[0]
        if q.dim() == 4:
            bq, nc, dim = q.shape[0], q.shape[2], q.shape[3]
        else:
            bq, nc, dim = q.shape
        be, k, row = rows.shape
        mul = 2 if model in fused.TWO_HALVES else 1
        n_q = 1 if model in fused.ONE_QUERY else 2
        if (nc != 1 or be not in (1, bq) or row != dim * mul or len(queries) != n_q or
                (rows.reg is not None and model != _REG_MODEL.get(rows.reg if isinstance(rows.reg, str) else "", "beta_kl")) or
                rows.ids.numel() != be * k):
            return None
        if any(t.dtype != torch.float32 or t.device != rows.device for t in queries):
            return None
        return dict(model=model, ids=rows.ids.reshape(be, k), q1=q, q2=queries[1] if n_q == 2 else None, gamma=gamma,
                    cen=cen, reg=rows.reg, b=bq)

    def score_lazy(self, model, rows, queries, gamma, cen):
        """Those logits in one launch of the fused scorer: [B, K], or [B, U, K] for 4-D queries (one slice per
        union branch, as the dense operators return it).  None when this is not a layout the fused scorer takes."""
        r = self.lazy_request(model, rows, queries, gamma, cen)
        if r is None:
            return None
        logit = self._score_branches(model, r["ids"], r["q1"], r["q2"], gamma, cen, r["reg"])
        if logit is None:
            return None
        return logit if r["q1"].dim() == 4 else logit[:, 0]

    def evaluate_pending(self, wanted):
        """Computes `wanted` (a LazyScores) together with every other pending one of this step that can share its
        launch: same model, margin, parameters, prologue and query tensors.  Their ids go side by side."""
        w = wanted.request

        def same(a, b):     # the same memory read the same way (the very tensor, or an equal view of it)
            if a is None or b is None:
                return a is b
            return a is b or (a.data_ptr() == b.data_ptr() and a.shape == b.shape and a.stride() == b.stride() and
                              a._version == b._version and a.requires_grad == b.requires_grad)

        alive = [p for p in (r() for r in self.pending_scores) if p is not None and p._value is None]
        group = [p for p in alive if p.request["model"] == w["model"] and
                 p.request["gamma"] == w["gamma"] and p.request["cen"] == w["cen"] and p.request["reg"] == w["reg"] and
                 same(p.request["q1"], w["q1"]) and same(p.request["q2"], w["q2"])]
        if not any(p is wanted for p in group):
            group.append(wanted)
        dev = self.sparse_embed.embedding.device
        # ids shared by the batch ([1, K], --share_negative) go into a launch of their own, K ids long; the per-query
        # ones ([B, K_i]) stand side by side in another
        shared = [p for p in group if p.request["ids"].shape[0] == 1 and w["b"] > 1]
        own = [p for p in group if not (p.request["ids"].shape[0] == 1 and w["b"] > 1)]
        for part in (own, shared):
            if not part:
                continue
            ids = [p.request["ids"].to(dev) for p in part]
            all_ids = ids[0] if len(ids) == 1 else torch.cat(ids, dim=1)
            # (union branches: the first maximal one, as torch.max(logit, dim=1) in the model code)
            values, index = self._score_max(w["model"], all_ids, w["q1"], w["q2"], w["gamma"], w["cen"], w["reg"])
            sizes = [i.shape[1] for i in ids]
            parts = [values] if len(ids) == 1 else torch.split(values, sizes, dim=1)
            iparts = [index] * len(ids) if (index is None or len(ids) == 1) else torch.split(index, sizes, dim=1)
            for p, val, ipart in zip(part, parts, iparts):
                # (each caller gets a tensor of its own layout, as torch.max would have returned it: .view() works)
                p._value = val.contiguous()
                p._index = None if ipart is None else ipart.contiguous()
        self.pending_scores = [r for r in self.pending_scores if r() is not None and r()._value is None]

    def score_negatives(self, model, ids, q1, q2=None, gamma=0.0, cen=0.0, regularizer=None):
        """Gather-fused logits [B,K]; q1/q2 are [B,dim] or [B,1,dim] and receive gradients.
        ids [B,K], or [1,K] for negatives shared by all queries of the batch (the --share_negative
        layout, online_sampler.py:155-157): every query then scores the same K entities.
        Union queries: q1/q2 of shape [B,U,dim] or [B,U,1,dim] (the merged branch embeddings of
        kg_reasoning.py:326) give max over the U branches of each branch's logit, as the last line of
        every custom_cal_logit does (box.py:163, vec.py:89, rotate.py:141, beta.py:307)."""
        return self._score_max(model, ids, q1, q2, gamma, cen, regularizer)[0]

    def _launch(self, model, ids, q1, q2, gamma, cen, regularizer):
        """One launch of the fused scorer.  Returns (b, branches, shared, scores, index): scores [B * branches, K]
        for one branch or for ids shared by the batch, else (union queries with their own ids) the maximum over the
        branches [B, K] with index [B, K], the branch that held it."""
        table = self.sparse_embed.embedding
        b = q1.shape[0]
        dim = q1.shape[-1]
        branches = q1.numel() // (b * dim)
        if q2 is not None and q2.shape != q1.shape:
            raise _lib.SmxError("the two query tensors must have the same shape")
        ids = ids.to(table.device)
        if ids.dim() != 2:
            raise _lib.SmxError("ids must be [B,K] or [1,K]")
        shared = ids.shape[0] == 1 and b * branches > 1     # every query row (every branch of every query) scores the same K ids
        if not shared and ids.shape[0] != b:
            raise _lib.SmxError("ids must be [B,K] or [1,K]")
        q1c = q1.reshape(b * branches, dim).contiguous()
        q2c = None if q2 is None else q2.reshape(b * branches, dim).contiguous()
        params = fused.score_params(gamma, cen, regularizer)
        self.stats["fused_launches"] += 1
        scores, index = _FusedScoreFunc.apply(self, self.dummy_tensor, model, ids.contiguous(), params, q1c, q2c,
                                              torch.is_grad_enabled(), branches)
        return b, branches, shared, scores, index

    def _score_max(self, model, ids, q1, q2, gamma, cen, regularizer):
        """(values [B, K], index [B, K] or None): the maximum over the union branches of each branch's logit and the
        first branch that holds it, as torch.max(logit, dim=1) of the custom_cal_logit bodies; one branch: the logits
        and None.  Queries with their own ids take the maximum inside the scorer; for ids shared by the batch the
        branch rows are scored like queries and torch.max runs on [B, U, K]."""
        b, branches, shared, scores, index = self._launch(model, ids, q1, q2, gamma, cen, regularizer)
        if branches == 1:
            return scores, None
        if shared:
            return torch.max(scores.view(b, branches, -1), dim=1)
        return scores, index

    def _score_branches(self, model, ids, q1, q2, gamma, cen, regularizer):
        """[B, branches, K] logits of every union branch of every query, for code that wants them before the maximum;
        None for union queries with their own ids, whose branches meet inside the scorer."""
        b = q1.shape[0]
        branches = q1.numel() // (b * q1.shape[-1])
        if branches > 1 and not (ids.dim() == 2 and ids.shape[0] == 1):
            return None
        b, branches, shared, scores, _ = self._launch(model, ids, q1, q2, gamma, cen, regularizer)
        return scores.view(b, branches, -1)

    def _raise_for(self, code):
        if code == 2:
            raise _lib.SmxError("the segment plan of this step is invalid (a sort workgroup gave up waiting)")
        if code != 0:
            raise IndexError("entity id out of range in a sparse lookup")

    def check_ids(self):
        """Raises if any lookup since the last check met an id outside the table (synchronises)."""
        self._flag_event = None
        code = int(self.err_flag.item())
        if code != 0:
            self.err_flag.zero_()
        self._raise_for(code)

    def poll_pending_id_check(self, wait=True):
        """Looks at the flag a finished step left in pinned host memory, if one is waiting (see
        _check_ids_one_step_late), and raises for it.  Called wherever the next step, or the end of training, passes
        by: zero_grad (only if the copy has already landed), the start of apply_grad -- also of one that has nothing
        to apply --, saving the table's state_dict."""
        if self._flag_event is not None:
            if not wait and not self._flag_event.query():
                return
            self._flag_event.synchronize()
            self._flag_event = None
            code = int(self._flag_host[0])
            if code != 0:
                self.err_flag.zero_()
                self._raise_for(code)

    def _check_ids_one_step_late(self):
        """The per-step check without draining the queue: this step's flag is copied to pinned host memory behind
        the update, and looked at when the next step reaches its apply_grad (before that update is applied) -- by
        then the copy has long finished, so the host keeps running ahead of the device.  The step that met the bad id
        has by then scored row 0 in its place: its loss and the gradients of the dense parameters are those of a wrong
        lookup (no table row was updated for the bad id).  check_ids() after the step, or check_ids_synchronously =
        True, fails before anything uses them."""
        self._flag_host.copy_(self.err_flag, non_blocking=True)
        self._flag_event = torch.cuda.Event()
        self._flag_event.record()

    def apply_grad(self, lr):
        """Unique-merge, segment sum and row update of everything recorded since zero_grad().  Pairs whose id
        lies outside the table never reach a row (the plan keeps them apart), and the lookup that met one raises
        IndexError as table[idx] does in the reference (embed_rw.py:74-75) -- with check_ids_every_step (default)
        from the apply_grad of the following step, so that no step waits for the device; check_ids() asks at once."""
        self.step += 1  # counts calls, also those without gradients (embed_optimizer.py:156)
        self.pending_scores = []    # logits that nothing used have no gradient and must not ride along later
        self.poll_pending_id_check()    # the previous step's flag, before this step's update is applied
        if not self.grad_list and not self.fused_list:
            return
        self._apply_grad(lr)
        if self.check_ids_synchronously:
            self.check_ids()
        elif self.check_ids_every_step:
            self._check_ids_one_step_late()

    def _apply_grad(self, lr):
        n_rows = self.sparse_embed.num_rows
        table = self.sparse_embed.embedding.detach()
        with torch.no_grad():
            if len(self.fused_list) == 1 and not self.grad_list:
                rec = self.fused_list[0]
                plan = fused.build_plan(rec["ids"], n_rows, err_flag=self.err_flag)
                if rec["shared"]:
                    self.update_shared(plan, rec, lr)
                else:
                    self.update_fused(plan, rec, lr)
                return
            idx_list = [i.reshape(-1).to(self.sparse_embed.device) for i, _ in self.grad_list]
            grad_list = [g.reshape(g.shape[0] if g.dim() == 2 else -1, g.shape[-1]).contiguous().float()
                         for _, g in self.grad_list]
            if self.fused_list and (len(self.fused_list) == 1 or self._one_entity_pass(self.fused_list)):
                # positives and negatives of one query batch (kg_reasoning.py:340-355), or records of several batches
                # scored in one step: one plan over all their ids, one entity pass that reads each record's own
                # scores / upstream gradients / sign codes against its own queries.
                # Negatives shared by the batch bring one gradient row per list position (each the sum over all
                # queries, formed by one workgroup per row) instead of B x K pairs.  Those rows, and the rows of the
                # step's plain lookups -- the anchor entities every query starts from (box.py:137), whose gradient
                # autograd has materialised -- go behind the pairs in the same plan: such a row is added to its
                # entity's gradient when the entity's row is finished.
                recs = sorted(self.fused_list, key=lambda r: r["fwd_idx"])   # forward order, whatever autograd's was
                own = [r for r in recs if not r["shared"]]
                shared = [r for r in recs if r["shared"]]
                n_shared = sum(r["ids"].numel() for r in shared)
                n_lookup = sum(g.shape[0] for g in grad_list)
                rows = None
                if n_shared:
                    rows = torch.empty((n_shared + n_lookup, table.shape[1]), dtype=torch.float32, device=table.device)
                    at = 0
                    for r in shared:
                        k = r["ids"].numel()
                        fused.score_backward_entity_shared(r["model"], table, r["ids"].reshape(-1), r["q1"], r["q2"],
                                                           r["score"], r["gscore"], r["params"], grad_rows=rows[at:at + k])
                        at += k
                    for g in grad_list:
                        rows[at:at + g.shape[0]].copy_(g)
                        at += g.shape[0]
                elif grad_list:
                    rows = grad_list[0] if len(grad_list) == 1 else torch.cat(grad_list, dim=0)
                flat = torch.cat([r["ids"].reshape(-1) for r in own] + [r["ids"].reshape(-1) for r in shared] + idx_list,
                                 dim=0)
                plan = fused.build_plan(flat, n_rows, err_flag=self.err_flag)
                if own:
                    self.update_fused_multi(plan, own, lr, grad_rows=rows)
                else:
                    self.update_from_plan(plan, rows, lr)
                return
            self.stats["per_record_merges"] += len(self.fused_list)
            for rec in self.fused_list:  # reduce each fused record to (distinct ids, summed rows) first
                plan = fused.build_plan(rec["ids"], n_rows, err_flag=self.err_flag)
                merged = torch.empty((plan.n_uniq, table.shape[1]), dtype=torch.float32, device=table.device)
                if rec["shared"]:
                    fused.score_backward_entity_shared(rec["model"], table, rec["ids"].reshape(-1), rec["q1"], rec["q2"],
                                                       rec["score"], rec["gscore"], rec["params"], plan=plan, merged=merged)
                else:
                    self._entity_pass(plan, [rec], merged=merged)
                idx_list.append(plan.uniq)
                grad_list.append(merged)
            # (a single record is used as it is: torch.cat would copy its gradient rows)
            flat = idx_list[0] if len(idx_list) == 1 else torch.cat(idx_list, dim=0)
            rows = grad_list[0] if len(grad_list) == 1 else torch.cat(grad_list, dim=0)
            plan = fused.build_plan(flat, n_rows, err_flag=self.err_flag)
            self.update_from_plan(plan, rows.contiguous(), lr)

    def _entity_pass(self, plan, recs, merged=None, m=None, v=None, adam=None, grad_rows=None):
        """The fused entity pass over the plan of the records' ids (per-query records of one query batch, in the
        order of the plan), then grad_rows: merged rows and / or the optimizer update."""
        table = self.sparse_embed.embedding.detach()
        first = recs[0]
        if len(recs) == 1 and grad_rows is None and first["branches"] == 1:
            fused.score_backward_entity(first["model"], plan, table, first["q1"], first["q2"], first["score"],
                                        first["gscore"], first["params"], merged=merged, m=m, v=v, adam=adam,
                                        codes=first["codes"])
            return
        # records of one query batch share its tensors; those of several batches (several forward calls in one step)
        # get the batches one after the other and each record its stretch of them
        batches, starts = [], []
        for r in recs:
            for i, b in enumerate(batches):
                if self._same_tensor(r["q1"], b["q1"]) and self._same_tensor(r["q2"], b["q2"]):
                    starts.append(i)
                    break
            else:
                batches.append(r)
                starts.append(len(batches) - 1)
        if len(batches) == 1:
            q1, q2 = first["q1"], first["q2"]
            sources = [(r["score"], r["gscore"], r["codes"]) + ((r["winner"],) if first["branches"] > 1 else ())
                       for r in recs]
        else:
            dim = first["q1"].shape[-1]
            rows = [b["q1"].numel() // (dim * first["branches"]) for b in batches]
            offs = [sum(rows[:i]) for i in range(len(rows))]
            q1 = torch.cat([b["q1"].reshape(-1, dim) for b in batches], dim=0)
            q2 = None if first["q2"] is None else torch.cat([b["q2"].reshape(-1, dim) for b in batches], dim=0)
            sources = [(r["score"], r["gscore"], r["codes"], r["winner"] if first["branches"] > 1 else None,
                        offs[starts[i]], rows[starts[i]]) for i, r in enumerate(recs)]
        fused.score_backward_entity_multi(first["model"], plan, table, q1, q2, sources, first["params"],
                                          merged=merged, m=m, v=v, adam=adam, grad_rows=grad_rows,
                                          branches=first["branches"])

    @staticmethod
    def _same_tensor(a, b):
        if a is None or b is None:
            return a is b
        return a.data_ptr() == b.data_ptr() and a.shape == b.shape and a._version == b._version

    @staticmethod
    def _one_entity_pass(recs):
        """True when the fused records can share one entity pass: same model, score parameters and number of union
        branches, sign codes for all per-query records or for none, few enough of those.  Their query batches may
        differ (records of several forward calls in one step, embed_optimizer.py:155-163 of the reference)."""
        own = [r for r in recs if not r["shared"]]
        if len(recs) < 2 or len(own) > _lib.MAX_PAIR_SOURCES:
            return False
        first = recs[0]

        def same_params(a, b):
            return all(getattr(a, f) == getattr(b, f) for f, _ in a._fields_)

        return (all(r["model"] == first["model"] and same_params(r["params"], first["params"]) and
                    r["branches"] == first["branches"] and (r["q2"] is None) == (first["q2"] is None) and
                    r["q1"].shape[-1] == first["q1"].shape[-1] for r in recs[1:]) and
                all((r["codes"] is None) == (own[0]["codes"] is None) for r in own[1:]))


class _RowOptimizer(EmbeddingOptimizer):
    """Shared body of the concrete optimizers: state buffers live on the SparseEmbedding under the
    reference's names (so they are part of its state_dict, embed_optimizer.py:190-197, 257-262,
    314-320) and every update is one fused pass over the plan."""
    kind = None            # key of fused.opt_params
    first_moment = None    # buffer name of the [N,row] first moment (Adam only)
    second_moment = None   # buffer name of the squared-gradient state, [N,row] or [N,1] with squeeze
    eps = 1e-8             # common/consts.py:20

    @classmethod
    def prepare_embed(cls, args, optim_mode, embed, fn_register):
        """State buffers under the reference's names (embed_optimizer.py:190-197, 257-262, 314-320), zero-filled,
        on the table's device; optim_mode[3] asks for one second-moment value per row."""
        table = embed.embedding.detach()
        squeeze = str(optim_mode[3]).lower() in ("true", "1") if len(optim_mode) > 3 else False
        if cls.first_moment and not hasattr(embed, cls.first_moment):
            fn_register(cls.first_moment, torch.zeros_like(table))
        if cls.second_moment and not hasattr(embed, cls.second_moment):
            shape = (table.shape[0], 1) if squeeze else tuple(table.shape)
            fn_register(cls.second_moment, torch.zeros(shape, dtype=table.dtype, device=table.device))

    def prepare_state(self):
        self.prepare_embed(self.args, self.optim_mode, self.sparse_embed, self.sparse_embed.register_tensor)

    def _state(self):
        emb = self.sparse_embed
        m = getattr(emb, self.first_moment) if self.first_moment else None
        v = getattr(emb, self.second_moment) if self.second_moment else None
        return m, v

    def _params(self, lr):
        return fused.opt_params(self.kind, lr, step=self.step, squeeze=self.squeeze, eps=self.eps)

    def update_from_plan(self, plan, grad_rows, lr):
        m, v = self._state()
        fused.rows_backward(plan, grad_rows, table=self.sparse_embed.embedding.detach(), m=m, v=v,
                            adam=self._params(lr))

    def update_fused_multi(self, plan, recs, lr, grad_rows=None):
        m, v = self._state()
        self._entity_pass(plan, recs, m=m, v=v, adam=self._params(lr), grad_rows=grad_rows)

    def update_shared(self, plan, rec, lr):
        m, v = self._state()
        fused.score_backward_entity_shared(rec["model"], self.sparse_embed.embedding.detach(), rec["ids"].reshape(-1),
                                           rec["q1"], rec["q2"], rec["score"], rec["gscore"], rec["params"], plan=plan,
                                           m=m, v=v, adam=self._params(lr))

    def update_fused(self, plan, rec, lr):
        m, v = self._state()
        self._entity_pass(plan, [rec], m=m, v=v, adam=self._params(lr))


class AdamEmbedOptimizer(_RowOptimizer):
    """Lazy Adam with one global step counter, betas (0.9, 0.999) (embed_optimizer.py:188-252)."""
    kind, first_moment, second_moment = "adam", "state_sum_fo", "state_sum_sq"


class SGDEmbedOptimizer(_RowOptimizer):
    """embed_optimizer.py:166-178."""
    kind = "sgd"


class AdaGradEmbedOptimizer(_RowOptimizer):
    """embed_optimizer.py:312-349."""
    kind, second_moment = "adagrad", "state_sum"


class RMSpropEmbedOptimizer(_RowOptimizer):
    """embed_optimizer.py:255-309 (alpha = 0.99)."""
    kind, second_moment = "rmsprop", "state_sum"


def get_optim_class(args):
    """embed_optimizer.py:352-364."""
    mode = args.optim_mode
    if isinstance(mode, str):
        mode = tuple(x.strip() for x in mode.strip("()").split(","))
    classes = {"adam": AdamEmbedOptimizer, "rmsprop": RMSpropEmbedOptimizer, "adagrad": AdaGradEmbedOptimizer,
               "sgd": SGDEmbedOptimizer}
    if mode[1] not in classes:
        raise NotImplementedError(mode[1])
    return classes[mode[1]]
