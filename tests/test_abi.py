"""CPU-side checks of the C ABI: the library loads and exports every symbol that
include/smore_amd.h declares, and the ctypes table covers the same set."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header="smore_amd.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(smx_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    from smore_amd import _lib
    names = _declared()
    assert len(names) >= 7
    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail("libsmore_amd.so is not built (run __graft_entry__.build())")
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == names


def test_measuring_entry_points_stay_out_of_the_drop_in_header():
    """include/smx_measure.h: exported by the same library, bound by the ctypes table of their own, absent from
    smore_amd.h."""
    from smore_amd import _lib
    names = _declared("smx_measure.h")
    assert names == sorted(_lib.MEASURE_SIGNATURES) and not set(names) & set(_declared())
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in smx_measure.h but not exported"


def test_probe_library_exports_its_header():
    """The benchmark's bandwidth probes live in a library of their own, outside the drop-in ABI."""
    from smore_amd import _lib
    if not os.path.exists(_lib.PROBE_PATH):
        pytest.fail("libsmx_probe.so is not built (run __graft_entry__.build())")
    lib = ctypes.CDLL(_lib.PROBE_PATH)
    for n in _declared("smx_probe.h"):
        assert hasattr(lib, n), f"{n} declared in smx_probe.h but not exported"
    assert not any("probe" in n for n in _declared())


def test_host_only_entry_points():
    from smore_amd import _lib
    lib = _lib.load()
    assert lib.smx_version() >= 1
    assert lib.smx_kind_from_name(b"box_out") == 2
    assert lib.smx_kind_from_name(b"beta_fisher_approx") == 9
    assert lib.smx_kind_from_name(b"nope") == -1
    assert lib.smx_set_option(_lib.OPTION_SERIAL_BACKWARD, 0) == 0 and lib.smx_set_option(99, 1) != 0
    assert lib.smx_set_option(2, 1) != 0, "the drop-in ABI has no switch that leaves a partial step behind"
    import ctypes as c
    opt = _lib.OptParams(1e-3, 0.9, 0.999, 1e-8, 2, _lib.OPT_KINDS["adam"], 0, None)
    out = (c.c_float * 2)()
    assert lib.smx_opt_step_consts(c.byref(opt), out) == 0
    assert abs(out[0] + 1e-3 / (1 - 0.9 ** 2)) < 1e-9 and abs(out[1] - (1 - 0.999 ** 2) ** -0.5) < 1e-4


def test_workspace_sizes_of_the_shared_negative_calls():
    """smx_shared_workspace_bytes (host only): the list's rows side by side [K, row] for every model (the query
    backward's copy; the same size as the entity side's sums [K, n_q dim] of the matrix-product models and as
    ComplEx's unit-length rows); BetaE its per-row terms [K, 2 dim + 1] and per-query terms [B]."""
    from smore_amd import _lib
    from smore_amd.fused import MODELS
    lib = _lib.load()
    b, k, d = 512, 1024, 400
    up = lambda n: (4 * n + 255) // 256 * 256
    for model, mul in (("l1", 1), ("l2", 1), ("box", 1), ("rotate", 2)):
        assert lib.smx_shared_workspace_bytes(MODELS[model], b, k, d) == up(k * mul * d)
    assert lib.smx_shared_workspace_bytes(MODELS["distmult"], b, k, d) == up(k * d)
    assert lib.smx_shared_workspace_bytes(MODELS["complex"], b, k, d) == up(k * 2 * d)
    assert lib.smx_shared_workspace_bytes(MODELS["beta_kl"], b, k, d) == up(k * (2 * d + 1) + b)
    assert lib.smx_shared_workspace_bytes(99, b, k, d) == 0


def test_multi_stream_entity_pass_refuses_bad_source_lists():
    """Argument checks of smx_score_backward_entity_multi happen before any launch: they can run without a GPU."""
    from smore_amd import _lib
    import ctypes as c
    lib = _lib.load()
    params = _lib.ScoreParams(24.0, 0.02, 0, 0.0, 0.0, 0.0)
    plan = _lib.PlanView(None, None, None, None, None, None, None, 40)
    src = (_lib.PairSource * 5)()
    fake = c.c_void_p(256)          # never dereferenced: every case below is refused on the host
    for i in range(5):
        src[i] = _lib.PairSource(fake, fake, None, 0, 4, None)
    call = lambda n_src, b=2, rows=None, n_rows=0: lib.smx_score_backward_entity_multi(
        2, None, c.byref(plan), fake, 100, fake, fake, c.cast(src, c.c_void_p), n_src, b, 8, c.byref(params), fake, None,
        None, None, fake, 1 << 20, rows, n_rows)
    assert call(0) != 0 and call(5) != 0
    assert b"pair sources" in lib.smx_last_error()
    assert call(2, b=7) != 0 and b"pairs" in lib.smx_last_error()          # 2 sources x 7 x 4 pairs, the plan holds 40
    src[1] = _lib.PairSource(fake, fake, fake, 64, 4, None)                       # sign codes for one source only
    assert call(2, b=5) != 0 and b"sign codes" in lib.smx_last_error()
    src[1] = _lib.PairSource(fake, None, None, 0, 4, None)
    assert call(2, b=5) != 0 and b"incomplete" in lib.smx_last_error()
    src[1] = _lib.PairSource(fake, fake, None, 0, 4, None)
    assert call(2, b=5, rows=fake, n_rows=0) != 0 and b"gradient rows" in lib.smx_last_error()
    assert call(2, b=5, rows=None, n_rows=3) != 0 and b"gradient rows" in lib.smx_last_error()
    assert call(2, b=5, rows=fake, n_rows=3) != 0 and b"gradient rows" in lib.smx_last_error()   # the plan holds 40, not 43


def test_scorer_refuses_tables_whose_ids_need_more_than_32_bits():
    """The forward finds equal ids of a tile by their low 32 bits: a table with more rows is refused on the host."""
    from smore_amd import _lib
    import ctypes as c
    lib = _lib.load()
    params = _lib.ScoreParams(24.0, 0.02, 0, 0.0, 0.0, 0.0)
    fake = c.c_void_p(256)          # never dereferenced
    rc = lib.smx_score_forward(2, None, fake, 1 << 32, fake, fake, fake, fake, 2, 4, 8, c.byref(params), None, None, 0)
    assert rc != 0 and b"wider than 32 bits" in lib.smx_last_error()


def test_entity_side_options_are_refused_where_a_model_has_none():
    """The clamp prologue belongs to beta_kl, unit-length rows to complex and distmult (complex.py:142-146); decided
    on the host, before any launch."""
    from smore_amd import _lib
    import ctypes as c
    lib = _lib.load()
    fake = c.c_void_p(256)          # never dereferenced
    fwd = lambda model, params: lib.smx_score_forward(model, None, fake, 100, fake, fake, fake, fake, 2, 4, 8,
                                                      c.byref(params), None, None, 0)
    assert fwd(2, _lib.ScoreParams(24.0, 0.02, 0, 0.0, 0.0, 0.0, 1)) != 0 and b"complex and distmult models only" in lib.smx_last_error()
    assert fwd(5, _lib.ScoreParams(0.0, 0.0, 1, 1.0, 0.05, 1e9, 0)) != 0 and b"beta_kl model only" in lib.smx_last_error()
    params = _lib.ScoreParams(24.0, 0.02, 0, 0.0, 0.0, 0.0, 1)
    rc = lib.smx_rank_answer_keys(2, None, fake, 100, fake, fake, 2, 8, c.byref(params), fake, fake, 4, fake, fake)
    assert rc != 0 and b"complex and distmult models only" in lib.smx_last_error()
    assert c.sizeof(_lib.ScoreParams) == 28      # seven four-byte fields, as the header declares them


def test_missing_library_fails_loudly(monkeypatch):
    from smore_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libsmore_amd.so")
    with pytest.raises(_lib.SmxError):
        _lib.load()
