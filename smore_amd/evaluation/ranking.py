"""Filtered ranks of the answers of a batch of queries among ALL entities, as test_step_mp computes
them (smore/training/train_process.py:112-160), on the streaming HIP scan instead of
`argsort` over the [1, nentity] logit row."""
import ctypes

import torch

from .. import _lib
from ..fused import MODELS, _dims, _ptr, _stream, _workspace

_TOP = -(1 << 63)  # flips the top bit: unsigned key order -> signed int64 order


def filtered_ranks(model, table, q1, q2, params, easy_answers, hard_answers, branches=1):
    """model: score model name; table [N,row]; q1/q2 [B,dim] (q2 None for l1/l2); params from
    fused.score_params (gamma, cen, regularizer); easy_answers / hard_answers: per query a sequence of
    entity ids (disjoint, train_process.py:139).  Returns per query a pair of int64 tensors (device):
    the filtered ranks (1-based) of its hard answers, in the order given, and of its easy answers.
    branches > 1: union queries, q1/q2 [B, branches, dim]; an entity's logit is the maximum over the branches
    (custom_cal_logit, box.py:163)."""
    if q1.numel() % (branches * q1.shape[-1]):
        raise _lib.SmxError("q1 must hold `branches` rows per query")
    b = q1.numel() // (branches * q1.shape[-1])
    if len(easy_answers) != b or len(hard_answers) != b:
        raise _lib.SmxError("one answer list per query is needed")
    n = table.shape[0]
    lists = [list(e) + list(h) for e, h in zip(easy_answers, hard_answers)]
    a = max(1, max(len(x) for x in lists))
    ids = torch.zeros((b, a), dtype=torch.int64)
    for i, x in enumerate(lists):
        if x:
            row = torch.as_tensor(x, dtype=torch.int64)
            if int(row.min()) < 0 or int(row.max()) >= n:
                raise IndexError("answer id outside the entity table")
            if row.unique().numel() != row.numel():
                raise _lib.SmxError("an entity is listed twice among the answers of one query")
            ids[i, : len(x)] = row
    counts = torch.tensor([len(x) for x in lists], dtype=torch.int32)
    dev = table.device
    ids, counts = ids.to(dev), counts.to(dev)
    q1c = q1.reshape(b * branches, -1).contiguous()
    q2c = None if q2 is None else q2.reshape(b * branches, -1).contiguous()
    _, _, dim = _dims(model, table, ids, q1c[:b], None if q2c is None else q2c[:b])
    scores = torch.empty((b, a), dtype=torch.float32, device=dev)
    keys = torch.empty((b, a), dtype=torch.int64, device=dev)  # holds the unsigned 64-bit keys bit for bit
    ranks = torch.empty((b, a), dtype=torch.int64, device=dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        _lib.call("smx_rank_answer_keys_union", MODELS[model], _stream(table), _ptr(table), n, _ptr(q1c), _ptr(q2c), b,
                  branches, dim, ctypes.byref(params), _ptr(ids), _ptr(counts), a, _ptr(scores), _ptr(keys))
        order = torch.argsort(keys ^ _TOP, dim=1, descending=True, stable=True)
        ids_sorted = torch.gather(ids, 1, order).contiguous()
        keys_sorted = torch.gather(keys, 1, order).contiguous()
        ws = _workspace(lib.smx_rank_workspace_bytes(b, a), dev)
        _lib.call("smx_rank_scan_union", MODELS[model], _stream(table), _ptr(table), n, _ptr(q1c), _ptr(q2c), b, branches,
                  dim, ctypes.byref(params), _ptr(ids_sorted), _ptr(keys_sorted), _ptr(counts), a, _ptr(ranks), _ptr(ws),
                  ws.numel())
    back = torch.empty_like(ranks)
    back.scatter_(1, order, ranks)  # rank of the answer in the slot it was given in
    out = []
    for i, (e, h) in enumerate(zip(easy_answers, hard_answers)):
        ne, nh = len(e), len(h)
        out.append((back[i, ne: ne + nh], back[i, :ne]))
    return out


def candidate_ranks(model, table, q1, q2, params, negative_sample, n_hard, err_flag=None, branches=1):
    """The other branch of test_step_mp (train_process.py:118-128, 141-147): the evaluation set brings its own
    candidates.  negative_sample [B, C] int64 on the table's device, -1 = padding; the first n_hard[b] candidates
    of query b are its hard answers (n_hard: sequence or int tensor of B counts).  Returns (negative_logit [B, C]
    with the -1e6 bias on the padding, ranking [B, C] int64, filtered ranks of the hard answers [B, max n_hard]
    int64, 0 in unused slots) -- one launch, no argsort.  branches > 1: union queries, q1/q2 [B, branches, dim],
    logits are the maximum over the branches."""
    if q1.numel() % (branches * q1.shape[-1]):
        raise _lib.SmxError("q1 must hold `branches` rows per query")
    b = q1.numel() // (branches * q1.shape[-1])
    if negative_sample.dim() != 2 or negative_sample.shape[0] != b or negative_sample.dtype != torch.int64:
        raise _lib.SmxError("negative_sample must be int64 [B, C]")
    dev = table.device
    cand = negative_sample.to(dev).contiguous()
    counts = torch.as_tensor(n_hard, dtype=torch.int32).reshape(-1)
    if counts.numel() != b or int(counts.min()) < 0 or int(counts.max()) > cand.shape[1]:
        raise _lib.SmxError("one hard-answer count per query, between 0 and C")
    h = max(1, int(counts.max()))
    counts = counts.to(dev)
    q1c = q1.reshape(b * branches, -1).contiguous()
    q2c = None if q2 is None else q2.reshape(b * branches, -1).contiguous()
    _, _, dim = _dims(model, table, cand, q1c[:b], None if q2c is None else q2c[:b])
    c = cand.shape[1]
    logit = torch.empty((b, c), dtype=torch.float32, device=dev)
    ranking = torch.empty((b, c), dtype=torch.int64, device=dev)
    hard = torch.empty((b, h), dtype=torch.int64, device=dev)
    with torch.cuda.device(dev):
        _lib.call("smx_rank_candidates_union", MODELS[model], _stream(table), _ptr(table), table.shape[0], _ptr(q1c),
                  _ptr(q2c), b, branches, dim, ctypes.byref(params), _ptr(cand), c, _ptr(counts), h, _ptr(logit),
                  _ptr(ranking), _ptr(hard), _ptr(err_flag))
    return logit, ranking, hard


def ranking_metrics(hard_ranks):
    """MRR, HITS1/3/10 and HITS1max of one query from the filtered ranks of its hard answers
    (train_process.py:146-152); an empty tensor gives zeros, as the reference does for a query whose
    answer is not among the candidates."""
    if hard_ranks.numel() == 0:
        return dict(MRR=0.0, HITS1=0.0, HITS3=0.0, HITS10=0.0, HITS1max=0.0)
    r = hard_ranks.to(torch.float32)
    return dict(MRR=float((1.0 / r).mean()), HITS1=float((r <= 1).float().mean()), HITS3=float((r <= 3).float().mean()),
                HITS10=float((r <= 10).float().mean()), HITS1max=float(r.min() == 1))
