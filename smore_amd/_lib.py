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
}

_lib = None


class SmxError(RuntimeError):
    pass


def load():
    """Returns the loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise SmxError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C smore_amd/csrc`. There is no fallback path.")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
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
