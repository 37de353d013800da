"""ctypes access to the C restatement ``ks_oracle_c.c`` (test infrastructure only)."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libks_oracle.so")


def build():
    subprocess.run(["make", "-C", _HERE, "-B"], check=True, capture_output=True)


def _load():
    if not os.path.exists(_SO):
        build()
    lib = ctypes.CDLL(_SO)
    for name in ("ks_oracle_factor_f32", "ks_oracle_factor_f64"):
        fn = getattr(lib, name)
        fn.restype = ctypes.c_int
        fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_long,
                       ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
    return lib


_lib = None


def factor(x, wk, pattern, bs_last):
    """``x``: float32/float64 (in, n) or (n, in); ``wk``: kernel format (a*d*c, b).
    Returns float64 output in the same layout, accumulated in double."""
    global _lib
    if _lib is None:
        _lib = _load()
    a, b, c, d = pattern
    x = np.ascontiguousarray(x)
    wk = np.ascontiguousarray(wk, dtype=x.dtype)
    assert x.dtype in (np.float32, np.float64)
    nb = x.shape[1] if bs_last else x.shape[0]
    assert (x.shape[0] if bs_last else x.shape[1]) == a * c * d
    assert wk.shape == (a * d * c, b)
    y = np.empty((a * b * d, nb) if bs_last else (nb, a * b * d), dtype=np.float64)
    fn = _lib.ks_oracle_factor_f32 if x.dtype == np.float32 else _lib.ks_oracle_factor_f64
    rc = fn(x.ctypes.data, wk.ctypes.data, y.ctypes.data, nb, a, b, c, d, int(bool(bs_last)))
    assert rc == 0
    return y
