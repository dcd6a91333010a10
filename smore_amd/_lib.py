"""ctypes binding of libsmore_amd.so (C ABI declared in include/smore_amd.h).

There is no CPU or eager fallback: if the library is missing, or a call
returns a non-zero status, the caller gets an exception.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsmore_amd.so")

_c = ctypes
_sz = _c.c_size_t
_vp = _c.c_void_p
_i = _c.c_int
_f = _c.c_float
_d = _c.c_double
_l = _c.c_long

_DENSE_FWD = [_i, _vp, _vp, _vp, _vp, _vp] + [_sz] * 7
_DENSE_BWD = [_i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp] + [_sz] * 7

# name -> (restype, argtypes); must list every symbol of include/smore_amd.h
SIGNATURES = {
    "smx_version": (_i, []),
    "smx_last_error": (_c.c_char_p, []),
    "smx_kind_from_name": (_i, [_c.c_char_p]),
    "smx_dist_forward_f32": (_i, _DENSE_FWD),
    "smx_dist_forward_f64": (_i, _DENSE_FWD),
    "smx_dist_backward_f32": (_i, _DENSE_BWD),
    "smx_dist_backward_f64": (_i, _DENSE_BWD),
    "smx_set_option": (_i, [_i, _i]),
    "smx_score_codes_bytes": (_sz, [_i, _sz, _sz]),
    # model, stream, table, n_rows, idx, q1, q2, score, B, K, dim, params, err_flag, codes, codes_bytes
    "smx_score_forward": (_i, [_i, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp, _vp, _vp, _sz]),
    # model, stream, table, n_rows, idx, q1, q2, score, gscore, gq1, gq2, B, K, dim, params, fwd_codes, bytes
    "smx_score_backward_query": (_i, [_i, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp, _vp,
                                      _sz]),
    "smx_shared_workspace_bytes": (_sz, [_i, _sz, _sz, _sz]),
    # model, stream, table, n_rows, ids, q1, q2, score, B, K, dim, params, err_flag, ws, ws_bytes
    "smx_score_forward_shared": (_i, [_i, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp, _vp, _vp, _sz]),
    # model, stream, table, n_rows, ids, q1, q2, score, gscore, gq1, gq2, B, K, dim, params, ws, ws_bytes
    "smx_score_backward_query_shared": (_i, [_i, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp,
                                             _vp, _sz]),
    # model, stream, table, n_rows, ids, q1, q2, score, gscore, B, K, dim, params, plan, grad_rows, merged, m, v, adam
    "smx_score_backward_entity_shared": (_i, [_i, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp, _vp, _vp,
                                              _vp, _vp, _vp, _vp, _vp, _sz]),
    "smx_union_workspace_bytes": (_sz, [_sz, _sz, _sz]),
    # model, stream, table, n_rows, idx, q1, q2, score, winner, B, U, K, dim, params, err_flag, ws, ws_bytes
    "smx_score_forward_union": (_i, [_i, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _vp, _vp, _vp, _sz]),
    # model, stream, table, n_rows, idx, q1, q2, score, gscore, winner, gq1, gq2, B, U, K, dim, params
    "smx_score_backward_query_union": (_i, [_i, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz,
                                            _vp]),
    # model, stream, plan, table, n_rows, q1, q2, src[], n_src, B, U, dim, params, merged, m, v, adam, ws, ws_bytes,
    # grad_rows, n_grad_rows
    "smx_score_backward_entity_union": (_i, [_i, _vp, _vp, _vp, _sz, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _vp, _vp, _vp, _vp,
                                             _vp, _vp, _sz, _vp, _sz]),
    "smx_plan_workspace_bytes": (_sz, [_sz, _sz]),
    # stream, idx, n_pairs, n_rows, ws, ws_bytes, order, sorted_ids, seg_of_pos, uniq, seg_start, inverse, pair_seg,
    # n_uniq, err
    "smx_plan_build": (_i, [_vp, _vp, _sz, _sz, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "smx_entity_workspace_bytes": (_sz, [_sz, _sz]),
    "smx_opt_step_consts": (_i, [_vp, _vp]),
    "smx_fused_workspace_bytes": (_sz, [_i, _sz, _sz]),
    # model, stream, plan, table, n_rows, q1, q2, score, gscore, B, K, dim, params, merged, m, v, adam, ws, ws_bytes,
    # fwd_codes, bytes
    "smx_score_backward_entity": (_i, [_i, _vp, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp, _vp, _vp, _vp,
                                       _vp, _vp, _sz, _vp, _sz]),
    # model, stream, plan, table, n_rows, q1, q2, src[], n_src, B, dim, params, merged, m, v, adam, ws, ws_bytes
    "smx_score_backward_entity_multi": (_i, [_i, _vp, _vp, _vp, _sz, _vp, _vp, _vp, _sz, _sz, _sz, _vp, _vp, _vp, _vp,
                                             _vp, _vp, _sz, _vp, _sz]),
    # model, stream, plan, table, n_rows, idx, q1, q2, score, gscore, gq1, gq2, B, K, dim, params, merged, m, v,
    # adam, ws, ws_bytes, fwd_codes, fwd_codes_bytes
    "smx_score_backward_fused": (_i, [_i, _vp, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp,
                                      _vp, _vp, _vp, _vp, _vp, _sz, _vp, _sz]),
    # stream, plan, grad_rows, row_len, merged, table, m, v, adam, ws, ws_bytes
    "smx_rank_workspace_bytes": (_sz, [_sz, _sz]),
    # model, stream, table, n_rows, q1, q2, B, dim, params, ans_id, ans_count, A, ans_score, ans_key
    "smx_rank_answer_keys": (_i, [_i, _vp, _vp, _sz, _vp, _vp, _sz, _sz, _vp, _vp, _vp, _sz, _vp, _vp]),
    # model, stream, table, n_rows, q1, q2, B, dim, params, ans_id, ans_key, ans_count, A, rank, ws, ws_bytes
    "smx_rank_scan": (_i, [_i, _vp, _vp, _sz, _vp, _vp, _sz, _sz, _vp, _vp, _vp, _vp, _sz, _vp, _vp, _sz]),
    # model, stream, table, n_rows, q1, q2, B, dim, params, cand, C, n_hard, H, logit, ranking, hard_rank, err
    "smx_rank_candidates": (_i, [_i, _vp, _vp, _sz, _vp, _vp, _sz, _sz, _vp, _vp, _sz, _vp, _sz, _vp, _vp, _vp, _vp]),
    # the same three with U (branch rows per query) behind B
    "smx_rank_answer_keys_union": (_i, [_i, _vp, _vp, _sz, _vp, _vp, _sz, _sz, _sz, _vp, _vp, _vp, _sz, _vp, _vp]),
    "smx_rank_scan_union": (_i, [_i, _vp, _vp, _sz, _vp, _vp, _sz, _sz, _sz, _vp, _vp, _vp, _vp, _sz, _vp, _vp, _sz]),
    "smx_rank_candidates_union": (_i, [_i, _vp, _vp, _sz, _vp, _vp, _sz, _sz, _sz, _vp, _vp, _sz, _vp, _sz, _vp, _vp, _vp,
                                       _vp]),
    "smx_sample_loss_workspace_bytes": (_sz, [_sz]),
    # stream, pos, neg, mask, weight, B, K, temperature, scale, out_loss, gpos, gneg, ws, ws_bytes
    "smx_sample_loss": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, ctypes.c_double, ctypes.c_double, _vp, _vp, _vp, _vp, _sz]),
    # stream, pos, neg, mask, weight, B, K, temperature, scale, out_loss, gpos, gneg
    "smx_sample_loss_static": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, ctypes.c_double, ctypes.c_double, _vp, _vp, _vp]),
    # stream, table, n_rows, row_len, idx, n, out, err
    "smx_gather_rows": (_i, [_vp, _vp, _sz, _sz, _vp, _sz, _vp, _vp]),
    "smx_rows_backward": (_i, [_vp, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _vp, _sz]),
}


class ScoreParams(ctypes.Structure):
    """smx_score_params of include/smore_amd.h."""
    _fields_ = [("gamma", _f), ("cen", _f), ("reg_on", _i), ("reg_add", _f), ("reg_lo", _f), ("reg_hi", _f),
                ("norm_on", _i)]


OPT_KINDS = {"adam": 1, "sgd": 2, "adagrad": 3, "rmsprop": 4}


class OptParams(ctypes.Structure):
    """smx_opt_params of include/smore_amd.h."""
    _fields_ = [("lr", _d), ("beta1", _d), ("beta2", _d), ("eps", _d), ("step", _l), ("kind", _i), ("squeeze", _i),
                ("step_consts_dev", _vp)]


class PlanView(ctypes.Structure):
    """smx_plan_view of include/smore_amd.h."""
    _fields_ = [("order", _vp), ("sorted_ids", _vp), ("seg_of_pos", _vp), ("seg_start", _vp), ("uniq", _vp),
                ("n_uniq", _vp), ("pair_seg", _vp), ("n_pairs", _sz)]



class PairSource(ctypes.Structure):
    """smx_pair_source of include/smore_amd.h."""
    _fields_ = [("score", _vp), ("gscore", _vp), ("fwd_codes", _vp), ("fwd_codes_bytes", _sz), ("K", _sz),
                ("winner", _vp), ("q_first", _sz), ("n_queries", _sz)]


MAX_PAIR_SOURCES = 4
OPTION_SERIAL_BACKWARD = 1

_lib = None
_probe = None
PROBE_PATH = os.path.join(_HERE, "libsmx_probe.so")


class SmxError(RuntimeError):
    pass


# measurement-only entry points of the same library (include/smx_measure.h), not part of the drop-in ABI
MEASURE_SIGNATURES = {
    # parts, then the arguments of smx_score_backward_fused
    "smx_measure_backward_fused": (_i, [_i] + SIGNATURES["smx_score_backward_fused"][1]),
    # the arguments of smx_plan_build, then spin_limit, force_abort
    "smx_measure_plan_build": (_i, SIGNATURES["smx_plan_build"][1] + [_c.c_uint, _i]),
    "smx_measure_query_kernel_events": (_i, [_vp, _vp]),
}


def load():
    """Returns the loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise SmxError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C smore_amd/csrc`. There is no fallback path.")
        lib = ctypes.CDLL(LIB_PATH)
        for table in (SIGNATURES, MEASURE_SIGNATURES):
            for name, (res, args) in table.items():
                fn = getattr(lib, name)
                fn.restype = res
                fn.argtypes = args
        _lib = lib
    return _lib


def check(rc):
    if rc != 0:
        msg = load().smx_last_error().decode("utf-8", "replace")
        raise SmxError(f"smore_amd status {rc}: {msg}")


def call(name, *args):
    check(getattr(load(), name)(*args))


def probe_bandwidth(kind, stream, a, b, nbytes, row_bytes, n_reads, sink):
    """smx_probe_bandwidth of libsmx_probe.so (include/smx_probe.h): the benchmark's bandwidth probes."""
    global _probe
    if _probe is None:
        if not os.path.exists(PROBE_PATH):
            raise SmxError(f"{PROBE_PATH} is missing: build it with `make -C smore_amd/csrc`")
        lib = ctypes.CDLL(PROBE_PATH)
        lib.smx_probe_bandwidth.restype = _i
        lib.smx_probe_bandwidth.argtypes = [_i, _vp, _vp, _vp, _sz, _sz, _sz, _vp]
        lib.smx_probe_last_error.restype = _c.c_char_p
        _probe = lib
    rc = _probe.smx_probe_bandwidth(kind, stream, a, b, nbytes, row_bytes, n_reads, sink)
    if rc != 0:
        raise SmxError(f"smx_probe status {rc}: {_probe.smx_probe_last_error().decode('utf-8', 'replace')}")
