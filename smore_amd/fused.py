"""Gather-fused scoring, segment plan and fused entity backward + sparse Adam.

Thin tensor-level front end of the fused entry points of libsmore_amd.so.  The
reference runs this as separate tensor programs: table[idx]
(smore/common/embedding/embed_rw.py:74-75), the distance operator
(smore/common/torchext/dist_func/*.py), gamma - dist (custom_cal_logit of
smore/models/*.py), and, after loss.backward(), unique / scatter-sum / Adam
(smore/common/embedding/embed_optimizer.py:39-48, 155-163, 208-252).
"""
import ctypes

import torch

from . import _lib

MODELS = {"l1": 0, "l2": 1, "box": 2, "rotate": 3, "beta_kl": 4, "complex": 5, "distmult": 6}
TWO_HALVES = ("rotate", "beta_kl", "complex")
ONE_QUERY = ("l1", "l2", "distmult")
SIMILARITY = ("complex", "distmult")     # logit = gamma + sim; the others: gamma - distance


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t):
    """The caller's current HIP stream on t's device, as an integer handle."""
    index = t.device.index
    if _raw_stream is not None and index is not None:      # (no Stream object built per call)
        return _raw_stream(index)
    return torch.cuda.current_stream(t.device).cuda_stream


class _Here:
    """`with _on(device):` when that device is already the current one: nothing to switch, nothing to restore."""

    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_here = _Here()


def _on(device):
    """torch.cuda.device(device), or nothing where the device is current already (the common case: a dozen library
    calls per step would otherwise each switch to the device they are on)."""
    if device.index is not None and torch.cuda.current_device() == device.index:
        return _here
    return torch.cuda.device(device)


def _ptr(t):
    return None if t is None else t.data_ptr()


def _f32(t, name):
    if t is None:
        return
    if t.dtype != torch.float32 or not t.is_contiguous() or t.device.type != "cuda":
        raise _lib.SmxError(f"{name} must be a contiguous fp32 device tensor")


def score_params(gamma, cen=0.0, regularizer=None, norm=False):
    """regularizer: None or (base_add, min_val, max_val) as in smore/common/modules.py:29-36.
    norm (complex), also spelled regularizer = "unit_halves": the halves of every entity row at unit length,
    smore/models/complex.py:142-146; (distmult), also regularizer = "unit_row": the whole row, distmult.py:129-130."""
    if isinstance(regularizer, str):
        if regularizer not in ("unit_halves", "unit_row"):
            raise _lib.SmxError(f"unknown entity option {regularizer!r}")
        regularizer, norm = None, True
    if regularizer is None:
        return _lib.ScoreParams(gamma, cen, 0, 0.0, 0.0, 0.0, 1 if norm else 0)
    add, lo, hi = regularizer
    return _lib.ScoreParams(gamma, cen, 1, add, lo, hi, 1 if norm else 0)


def new_error_flag(device):
    """Device int the kernels set to 1 when they meet an entity id outside the table."""
    return torch.zeros(1, dtype=torch.int32, device=device)


def _dims(model, table, idx, q1, q2):
    if model not in MODELS:
        raise _lib.SmxError(f"unknown score model {model}")
    _f32(table, "table")
    _f32(q1, "q1")
    _f32(q2, "q2")
    if (q2 is None) != (model in ONE_QUERY):
        raise _lib.SmxError(f"model {model} takes {'one' if model in ONE_QUERY else 'two'} query tensor(s)")
    mul = 2 if model in TWO_HALVES else 1
    b, dim = q1.shape[0], q1.shape[-1]
    if q1.numel() != b * dim or (q2 is not None and q2.shape != q1.shape):
        raise _lib.SmxError("query tensors must be [B, dim] (or [B, 1, dim])")
    if table.dim() != 2 or table.shape[1] != dim * mul:
        raise _lib.SmxError(f"table row length {tuple(table.shape)} does not match dim {dim} x {mul}")
    if idx is not None:
        if idx.dtype != torch.int64 or not idx.is_contiguous() or idx.device != table.device:
            raise _lib.SmxError("idx must be a contiguous int64 tensor on the table's device")
        if idx.dim() != 2 or idx.shape[0] != b:
            raise _lib.SmxError("idx must be [B, K]")
        k = idx.shape[1]
    else:
        if table.shape[0] % b:
            raise _lib.SmxError("dense rows must be [B*K, row]")
        k = table.shape[0] // b
    return b, k, dim


def new_codes(model, table, idx, q1):
    """Buffer for the sign codes of one step (see smx_score_codes_bytes), or None when the model or the
    row length has none.  Pass it to score_forward and, unchanged, to score_backward_fused."""
    if model not in MODELS:
        raise _lib.SmxError(f"unknown score model {model}")
    n_pairs = idx.numel() if idx is not None else table.shape[0]
    nbytes = _lib.load().smx_score_codes_bytes(MODELS[model], n_pairs, q1.shape[-1])
    return torch.empty(nbytes, dtype=torch.uint8, device=table.device) if nbytes else None


def score_forward(model, table, idx, q1, q2, params, err_flag=None, codes=None):
    """logit[b,k] = gamma - dist(table[idx[b,k]], q[b]).  idx None: table is the dense [B*K, row] rows.
    codes: buffer from new_codes() that receives the step's sign codes."""
    b, k, dim = _dims(model, table, idx, q1, q2)
    score = torch.empty((b, k), dtype=torch.float32, device=table.device)
    with _on(table.device):
        _lib.call("smx_score_forward", MODELS[model], _stream(table), _ptr(table), table.shape[0], _ptr(idx),
                  _ptr(q1), _ptr(q2), _ptr(score), b, k, dim, ctypes.byref(params), _ptr(err_flag),
                  _ptr(codes), 0 if codes is None else codes.numel())
    return score


def score_backward_query(model, table, idx, q1, q2, score, gscore, params, codes=None):
    """Gradients of sum(gscore * score) w.r.t. q1 (and q2).  codes: what score_forward saved (optional)."""
    b, k, dim = _dims(model, table, idx, q1, q2)
    _f32(score, "score")
    _f32(gscore, "gscore")
    gq1 = torch.empty_like(q1)
    gq2 = None if q2 is None else torch.empty_like(q2)
    with _on(table.device):
        _lib.call("smx_score_backward_query", MODELS[model], _stream(table), _ptr(table), table.shape[0], _ptr(idx),
                  _ptr(q1), _ptr(q2), _ptr(score), _ptr(gscore), _ptr(gq1), _ptr(gq2), b, k, dim,
                  ctypes.byref(params), _ptr(codes), 0 if codes is None else codes.numel())
    return gq1, gq2


def _shared_dims(model, table, ids, q1, q2):
    if model not in MODELS:
        raise _lib.SmxError(f"unknown score model {model}")
    _f32(table, "table")
    _f32(q1, "q1")
    _f32(q2, "q2")
    if (q2 is None) != (model in ONE_QUERY):
        raise _lib.SmxError(f"model {model} takes {'one' if model in ONE_QUERY else 'two'} query tensor(s)")
    mul = 2 if model in TWO_HALVES else 1
    b, dim = q1.shape[0], q1.shape[-1]
    if q1.numel() != b * dim or (q2 is not None and q2.shape != q1.shape):
        raise _lib.SmxError("query tensors must be [B, dim] (or [B, 1, dim])")
    if table.dim() != 2 or table.shape[1] != dim * mul:
        raise _lib.SmxError(f"table row length {tuple(table.shape)} does not match dim {dim} x {mul}")
    if ids.dtype != torch.int64 or not ids.is_contiguous() or ids.device != table.device or ids.numel() == 0:
        raise _lib.SmxError("shared ids must be a contiguous int64 tensor [K] (or [1, K]) on the table's device")
    return b, ids.numel(), dim


def _shared_workspace(model, b, k, dim, device, use):
    nbytes = _lib.load().smx_shared_workspace_bytes(MODELS[model], b, k, dim) if use else 0
    return _workspace(nbytes, device) if nbytes else None


def score_forward_shared(model, table, ids, q1, q2, params, err_flag=None, per_row_terms=True):
    """logit[b,k] = gamma - dist(table[ids[k]], q[b]) for K ids that every query scores (--share_negative).
    per_row_terms=False keeps beta_kl on the per-pair kernels (no workspace for the rows' terms; for comparison)."""
    b, k, dim = _shared_dims(model, table, ids, q1, q2)
    score = torch.empty((b, k), dtype=torch.float32, device=table.device)
    with _on(table.device):
        ws = _shared_workspace(model, b, k, dim, table.device, per_row_terms)
        _lib.call("smx_score_forward_shared", MODELS[model], _stream(table), _ptr(table), table.shape[0], _ptr(ids),
                  _ptr(q1), _ptr(q2), _ptr(score), b, k, dim, ctypes.byref(params), _ptr(err_flag), _ptr(ws),
                  0 if ws is None else ws.numel())
    return score


def score_backward_query_shared(model, table, ids, q1, q2, score, gscore, params, per_row_terms=True):
    """Gradients of sum(gscore * score) w.r.t. q1 (and q2) for shared ids."""
    b, k, dim = _shared_dims(model, table, ids, q1, q2)
    _f32(score, "score")
    _f32(gscore, "gscore")
    gq1 = torch.empty_like(q1)
    gq2 = None if q2 is None else torch.empty_like(q2)
    with _on(table.device):
        ws = _shared_workspace(model, b, k, dim, table.device, per_row_terms)
        _lib.call("smx_score_backward_query_shared", MODELS[model], _stream(table), _ptr(table), table.shape[0],
                  _ptr(ids), _ptr(q1), _ptr(q2), _ptr(score), _ptr(gscore), _ptr(gq1), _ptr(gq2), b, k, dim,
                  ctypes.byref(params), _ptr(ws), 0 if ws is None else ws.numel())
    return gq1, gq2


def score_backward_entity_shared(model, table, ids, q1, q2, score, gscore, params, plan=None, grad_rows=None,
                                 merged=None, m=None, v=None, adam=None, per_row_terms=True):
    """Entity side of shared ids (see smx_score_backward_entity_shared).  plan None: returns (and fills) grad_rows
    [K, row], one gradient row per list position.  plan (built over exactly these ids): merged rows per distinct id
    and / or the optimizer update of table, m, v in place."""
    b, k, dim = _shared_dims(model, table, ids, q1, q2)
    for t, name in ((score, "score"), (gscore, "gscore"), (grad_rows, "grad_rows"), (merged, "merged"), (m, "m"), (v, "v")):
        _f32(t, name)
    if score.shape != (b, k) or gscore.shape != (b, k):
        raise _lib.SmxError("score and gscore must be [B, K]")
    row_len = table.shape[1]
    if plan is None:
        if grad_rows is None:
            grad_rows = torch.empty((k, row_len), dtype=torch.float32, device=table.device)
        elif grad_rows.shape != (k, row_len):
            raise _lib.SmxError("grad_rows must be [K, row]")
    else:
        if plan.n_pairs != k:
            raise _lib.SmxError("the plan must be built over the shared ids")
        _check_state(table, m, v, adam)
        if merged is not None and (merged.dim() != 2 or merged.shape[1] != row_len):
            raise _lib.SmxError("merged must be [n_uniq or more, row]")
    with _on(table.device):
        view = None if plan is None else plan.view()
        ws = _shared_workspace(model, b, k, dim, table.device, per_row_terms)
        _lib.call("smx_score_backward_entity_shared", MODELS[model], _stream(table), _ptr(table), table.shape[0],
                  _ptr(ids), _ptr(q1), _ptr(q2), _ptr(score), _ptr(gscore), b, k, dim, ctypes.byref(params),
                  None if view is None else ctypes.byref(view), _ptr(grad_rows), _ptr(merged), _ptr(m), _ptr(v),
                  None if adam is None else ctypes.byref(adam), _ptr(ws), 0 if ws is None else ws.numel())
    return grad_rows


def gather_rows(table, idx, err_flag=None):
    """rows = table[idx] (idx any shape, flattened) -> [idx.numel(), row]."""
    _f32(table, "table")
    if idx.dtype != torch.int64 or idx.device != table.device:
        raise _lib.SmxError("idx must be an int64 tensor on the table's device")
    flat = idx.reshape(-1).contiguous()
    out = torch.empty((flat.numel(), table.shape[1]), dtype=torch.float32, device=table.device)
    if flat.numel():
        with _on(table.device):
            _lib.call("smx_gather_rows", _stream(table), _ptr(table), table.shape[0], table.shape[1], _ptr(flat),
                      flat.numel(), _ptr(out), _ptr(err_flag))
    return out


class SegmentPlan:
    """Device-resident result of grouping one step's pairs by entity id (see smx_plan_build)."""

    def __init__(self, n_pairs, n_rows, device, want_inverse):
        i32 = dict(dtype=torch.int32, device=device)
        self.n_pairs, self.n_rows = n_pairs, n_rows
        self.order = torch.empty(n_pairs, **i32)
        self.sorted_ids = torch.empty(n_pairs, **i32)
        self.seg_of_pos = torch.empty(n_pairs, **i32)
        self.seg_start = torch.empty(n_pairs + 1, **i32)
        self.uniq_buf = torch.empty(n_pairs, dtype=torch.int64, device=device)
        self.inverse = torch.empty(n_pairs, dtype=torch.int64, device=device) if want_inverse else None
        self.pair_seg = torch.empty(n_pairs, **i32)
        self.n_uniq_dev = torch.zeros(1, **i32)
        self._n_uniq = None

    @property
    def n_uniq(self):
        """Number of distinct ids (first use synchronises with the device)."""
        if self._n_uniq is None:
            n = int(self.n_uniq_dev.item())
            if n < 0:
                raise _lib.SmxError("the segment plan is invalid (a sort workgroup gave up waiting)")
            self._n_uniq = n
        return self._n_uniq

    @property
    def uniq(self):
        return self.uniq_buf[: self.n_uniq]

    def view(self):
        return _lib.PlanView(_ptr(self.order), _ptr(self.sorted_ids), _ptr(self.seg_of_pos), _ptr(self.seg_start),
                             _ptr(self.uniq_buf), _ptr(self.n_uniq_dev), _ptr(self.pair_seg), self.n_pairs)


def _workspace(nbytes, device):
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


def build_plan(idx, n_rows, want_inverse=False, err_flag=None, measure=None):
    """Sorts the pairs of idx (any shape, int64, device) by entity id; see SegmentPlan.
    measure (tests only): (spin_limit, force_abort) for smx_measure_plan_build (include/smx_measure.h)."""
    if idx.dtype != torch.int64 or idx.device.type != "cuda":
        raise _lib.SmxError("idx must be an int64 device tensor")
    flat = idx.reshape(-1).contiguous()
    n = flat.numel()
    plan = SegmentPlan(n, n_rows, flat.device, want_inverse)
    with _on(flat.device):
        nbytes = _lib.load().smx_plan_workspace_bytes(n, n_rows)
        if nbytes == 0:
            raise _lib.SmxError("smx_plan_workspace_bytes failed")
        ws = _workspace(nbytes, flat.device)
        entry, extra = ("smx_plan_build", ()) if measure is None else ("smx_measure_plan_build", tuple(measure))
        _lib.call(entry, _stream(flat), _ptr(flat), n, n_rows, _ptr(ws), ws.numel(), _ptr(plan.order),
                  _ptr(plan.sorted_ids), _ptr(plan.seg_of_pos), _ptr(plan.uniq_buf), _ptr(plan.seg_start),
                  _ptr(plan.inverse), _ptr(plan.pair_seg), _ptr(plan.n_uniq_dev), _ptr(err_flag), *extra)
    return plan


def adam_params(lr, step, beta1=0.9, beta2=0.999, eps=1e-8, squeeze=False, step_consts=None):
    """step_consts: device tensor of two floats kept up to date with set_step_consts(); the kernels then take
    the learning rate and the bias corrections from it at run time (needed when the launch is replayed
    from a HIP graph: its by-value arguments are frozen at capture)."""
    return _lib.OptParams(lr, beta1, beta2, eps, int(step), _lib.OPT_KINDS["adam"], int(bool(squeeze)),
                          _ptr(step_consts))


def opt_params(kind, lr, step=1, squeeze=False, eps=1e-8, alpha=0.99, step_consts=None):
    """Parameters of a row optimizer: kind in {adam, sgd, adagrad, rmsprop} (see smx_opt_params)."""
    if kind == "adam":
        return adam_params(lr, step, eps=eps, squeeze=squeeze, step_consts=step_consts)
    if kind not in _lib.OPT_KINDS:
        raise _lib.SmxError(f"unknown optimizer {kind}")
    return _lib.OptParams(lr, 0.0, alpha, eps, int(step), _lib.OPT_KINDS[kind], int(bool(squeeze)), _ptr(step_consts))


def set_step_consts(buf, opt):
    """Writes the per-step constants of `opt` (its lr and step) into the two-float device tensor `buf`, in
    stream order (a 8-byte copy from pinned memory)."""
    host = (ctypes.c_float * 2)()
    _lib.call("smx_opt_step_consts", ctypes.byref(opt), host)
    pinned = torch.tensor([host[0], host[1]], dtype=torch.float32).pin_memory()
    buf.copy_(pinned, non_blocking=True)
    return buf


def _check_state(table, m, v, opt):
    if m is not None and m.shape != table.shape:
        raise _lib.SmxError("the first-moment table must have the entity table's shape")
    if v is not None:
        want = table.shape[0] if (opt is not None and opt.squeeze) else table.numel()
        if v.numel() != want:
            raise _lib.SmxError("the second-moment table must be [N, row], or [N] / [N,1] with squeeze")


def score_backward_entity(model, plan, table, q1, q2, score, gscore, params, merged=None, m=None, v=None, adam=None,
                          codes=None):
    """Segmented entity gradient of sum(gscore * score); writes merged [>=U, row] and/or applies lazy Adam
    to table, m, v in place (all of the table's shape).  codes: what score_forward saved (optional)."""
    b, dim = q1.shape[0], q1.shape[-1]
    k = plan.n_pairs // b
    if model not in MODELS:
        raise _lib.SmxError(f"unknown score model {model}")
    for t, name in ((table, "table"), (q1, "q1"), (q2, "q2"), (score, "score"), (gscore, "gscore"),
                    (merged, "merged"), (m, "m"), (v, "v")):
        _f32(t, name)
    row_len = table.shape[1]
    _check_state(table, m, v, adam)
    if merged is not None and (merged.dim() != 2 or merged.shape[1] != row_len):
        raise _lib.SmxError("merged must be [n_uniq or more, row]")
    with _on(table.device):
        ws = _workspace(_lib.load().smx_entity_workspace_bytes(plan.n_pairs, row_len), table.device)
        view = plan.view()
        _lib.call("smx_score_backward_entity", MODELS[model], _stream(table), ctypes.byref(view), _ptr(table),
                  table.shape[0], _ptr(q1), _ptr(q2), _ptr(score), _ptr(gscore), b, k, dim, ctypes.byref(params),
                  _ptr(merged), _ptr(m), _ptr(v), None if adam is None else ctypes.byref(adam), _ptr(ws), ws.numel(),
                  _ptr(codes), 0 if codes is None else codes.numel())


def score_forward_union(model, table, idx, q1, q2, params, branches, err_flag=None):
    """Union queries: q1 / q2 [B * branches, dim] (a query's branch rows adjacent), idx [B, K].  Returns
    (score [B, K] = the maximum over the branches, winner [B, K] uint8 = the first branch that holds it)."""
    if model not in MODELS:
        raise _lib.SmxError(f"unknown score model {model}")
    _f32(table, "table")
    _f32(q1, "q1")
    _f32(q2, "q2")
    dim = q1.shape[-1]
    bu = q1.numel() // dim
    if bu % branches or idx.dim() != 2 or idx.shape[0] * branches != bu or idx.dtype != torch.int64 or \
            not idx.is_contiguous() or idx.device != table.device:
        raise _lib.SmxError("union scoring takes idx [B, K] int64 and query tensors [B * branches, dim]")
    b, k = idx.shape
    score = torch.empty((b, k), dtype=torch.float32, device=table.device)
    winner = torch.empty((b, k), dtype=torch.uint8, device=table.device)
    with _on(table.device):
        ws = _workspace(_lib.load().smx_union_workspace_bytes(b, branches, k), table.device)
        _lib.call("smx_score_forward_union", MODELS[model], _stream(table), _ptr(table), table.shape[0], _ptr(idx),
                  _ptr(q1), _ptr(q2), _ptr(score), _ptr(winner), b, branches, k, dim, ctypes.byref(params),
                  _ptr(err_flag), _ptr(ws), ws.numel())
    return score, winner


def score_backward_query_union(model, table, idx, q1, q2, score, gscore, winner, params, branches):
    """Gradients of sum(gscore * score) w.r.t. the branch rows q1 (and q2), [B * branches, dim]."""
    _f32(score, "score")
    _f32(gscore, "gscore")
    b, k = idx.shape
    dim = q1.shape[-1]
    gq1 = torch.empty_like(q1)
    gq2 = None if q2 is None else torch.empty_like(q2)
    with _on(table.device):
        _lib.call("smx_score_backward_query_union", MODELS[model], _stream(table), _ptr(table), table.shape[0], _ptr(idx),
                  _ptr(q1), _ptr(q2), _ptr(score), _ptr(gscore), _ptr(winner), _ptr(gq1), _ptr(gq2), b, branches, k,
                  dim, ctypes.byref(params))
    return gq1, gq2


def score_backward_entity_multi(model, plan, table, q1, q2, sources, params, merged=None, m=None, v=None, adam=None,
                                grad_rows=None, branches=1):
    """score_backward_entity for several index streams of one query batch (see smx_score_backward_entity_multi).
    sources: list of (score [B,K_s], gscore [B,K_s], codes or None[, winner[, q_first, n_queries]]); plan: built over
    the concatenation of the streams' flattened ids in the same order.  grad_rows [n, row]: materialised gradient rows
    of the step's plain lookups, whose ids are the last n entries of that concatenation.  branches > 1: union queries,
    q1 / q2 are [B * branches, dim] and every source brings its winner array (smx_score_backward_entity_union).
    Sources of different query batches: q1 / q2 hold the batches one after the other and a source names its stretch
    of queries with q_first and n_queries (its score is then [n_queries, K_s])."""
    dim = q1.shape[-1]
    b = q1.numel() // (dim * branches)
    if model not in MODELS:
        raise _lib.SmxError(f"unknown score model {model}")
    if not 1 <= len(sources) <= _lib.MAX_PAIR_SOURCES:
        raise _lib.SmxError(f"1 to {_lib.MAX_PAIR_SOURCES} pair sources")
    for t, name in ((table, "table"), (q1, "q1"), (q2, "q2"), (merged, "merged"), (m, "m"), (v, "v")):
        _f32(t, name)
    arr = (_lib.PairSource * len(sources))()
    for i, src in enumerate(sources):
        score, gscore, codes = src[:3]
        winner = src[3] if len(src) > 3 else None
        q_first, n_q = (int(src[4]), int(src[5])) if len(src) > 5 else (0, b)
        _f32(score, "score")
        _f32(gscore, "gscore")
        if n_q < 1 or q_first < 0 or q_first + n_q > b:
            raise _lib.SmxError(f"a source's queries {q_first} .. {q_first + n_q} of {b}")
        if score.numel() % n_q or gscore.shape != score.shape:
            raise _lib.SmxError("score and gscore of a source must both be [its queries, K]")
        if branches > 1 and winner is None:
            raise _lib.SmxError("union queries bring a winner array per source")
        if branches == 1:
            winner = None       # a union of one branch is a plain query: its winner array holds zeros
        arr[i] = _lib.PairSource(_ptr(score), _ptr(gscore), _ptr(codes), 0 if codes is None else codes.numel(),
                                 score.numel() // n_q, _ptr(winner), q_first, 0 if n_q == b else n_q)
    row_len = table.shape[1]
    _check_state(table, m, v, adam)
    if merged is not None and (merged.dim() != 2 or merged.shape[1] != row_len):
        raise _lib.SmxError("merged must be [n_uniq or more, row]")
    n_grad = 0
    if grad_rows is not None:
        _f32(grad_rows, "grad_rows")
        if grad_rows.dim() != 2 or grad_rows.shape[1] != row_len or grad_rows.shape[0] == 0:
            raise _lib.SmxError("grad_rows must be [n >= 1, row]")
        n_grad = grad_rows.shape[0]
    with _on(table.device):
        ws = _workspace(_lib.load().smx_entity_workspace_bytes(plan.n_pairs, row_len), table.device)
        view = plan.view()
        if branches > 1:
            _lib.call("smx_score_backward_entity_union", MODELS[model], _stream(table), ctypes.byref(view), _ptr(table),
                      table.shape[0], _ptr(q1), _ptr(q2), ctypes.cast(arr, ctypes.c_void_p), len(sources), b, branches,
                      dim, ctypes.byref(params), _ptr(merged), _ptr(m), _ptr(v),
                      None if adam is None else ctypes.byref(adam), _ptr(ws), ws.numel(), _ptr(grad_rows), n_grad)
        else:
            _lib.call("smx_score_backward_entity_multi", MODELS[model], _stream(table), ctypes.byref(view), _ptr(table),
                      table.shape[0], _ptr(q1), _ptr(q2), ctypes.cast(arr, ctypes.c_void_p), len(sources), b, dim,
                      ctypes.byref(params), _ptr(merged), _ptr(m), _ptr(v),
                      None if adam is None else ctypes.byref(adam), _ptr(ws), ws.numel(), _ptr(grad_rows), n_grad)


def score_backward_fused(model, plan, table, idx, q1, q2, score, gscore, params, merged=None, m=None, v=None,
                         adam=None, sign_codes=True, codes=None, measure_parts=None):
    """Query gradients and all entity rows of the step in one call (see smx_score_backward_fused).
    Returns (gq1, gq2); merged / table, m, v are written in place as in score_backward_entity.
    codes: the buffer score_forward filled for these pairs (table and queries unchanged since).
    sign_codes=False gives the call only the entity pass's own workspace, which keeps the box model on
    the path that re-reads the query rows (same results; for tests and comparison).
    measure_parts (1 or 2; benchmarks only): launch one half of the call through the measuring entry point
    smx_measure_backward_fused (include/smx_measure.h); the step such a call leaves is incomplete."""
    b, k, dim = _dims(model, table, idx, q1, q2)
    for t, name in ((score, "score"), (gscore, "gscore"), (merged, "merged"), (m, "m"), (v, "v")):
        _f32(t, name)
    if plan.n_pairs != b * k:
        raise _lib.SmxError("plan does not belong to these ids")
    _check_state(table, m, v, adam)
    if merged is not None and (merged.dim() != 2 or merged.shape[1] != table.shape[1]):
        raise _lib.SmxError("merged must be [n_uniq or more, row]")
    gq1 = torch.empty_like(q1)
    gq2 = None if q2 is None else torch.empty_like(q2)
    with _on(table.device):
        ws_bytes = _lib.load().smx_fused_workspace_bytes(MODELS[model], plan.n_pairs, dim) \
            if sign_codes and codes is None else \
            _lib.load().smx_entity_workspace_bytes(plan.n_pairs, table.shape[1])
        ws = _workspace(ws_bytes, table.device)
        view = plan.view()
        entry = ("smx_score_backward_fused",) if measure_parts is None else ("smx_measure_backward_fused", measure_parts)
        _lib.call(*entry, MODELS[model], _stream(table), ctypes.byref(view), _ptr(table),
                  table.shape[0], _ptr(idx), _ptr(q1), _ptr(q2), _ptr(score), _ptr(gscore), _ptr(gq1), _ptr(gq2),
                  b, k, dim, ctypes.byref(params), _ptr(merged), _ptr(m), _ptr(v),
                  None if adam is None else ctypes.byref(adam), _ptr(ws), ws.numel(),
                  _ptr(codes), 0 if codes is None else codes.numel())
    return gq1, gq2


def rows_backward(plan, grad_rows, merged=None, table=None, m=None, v=None, adam=None):
    """Segment sum of materialised gradient rows [P, row] (pair order) and optional lazy Adam."""
    for t, name in ((grad_rows, "grad_rows"), (merged, "merged"), (table, "table"), (m, "m"), (v, "v")):
        _f32(t, name)
    if grad_rows.dim() != 2 or grad_rows.shape[0] != plan.n_pairs:
        raise _lib.SmxError("grad_rows must be [P, row]")
    row_len = grad_rows.shape[1]
    if table is not None:
        _check_state(table, m, v, adam)
    with _on(grad_rows.device):
        ws = _workspace(_lib.load().smx_entity_workspace_bytes(plan.n_pairs, row_len), grad_rows.device)
        view = plan.view()
        _lib.call("smx_rows_backward", _stream(grad_rows), ctypes.byref(view), _ptr(grad_rows), row_len, _ptr(merged),
                  _ptr(table), _ptr(m), _ptr(v), None if adam is None else ctypes.byref(adam), _ptr(ws), ws.numel())
