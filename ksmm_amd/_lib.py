"""ctypes binding of libksmm_hip.so (the C ABI declared in include/ksmm_hip.h).

The library is built in-tree by ``python -m ksmm_amd.build``; loading fails loudly if it is
missing: there is no CPU or eager-PyTorch stand-in for ``algo='kernel'``.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libksmm_hip.so")

KSMM_F32, KSMM_F16, KSMM_FP8_E4M3 = 0, 1, 2
ALGO_AUTO, ALGO_GENERIC, ALGO_WAVE, ALGO_TILE = 0, 1, 2, 3
MAX_FACTORS = 16
ACT_NONE, ACT_GELU = 0, 1
ABI_VERSION = 2

c_i64 = ctypes.c_int64
c_int = ctypes.c_int
c_vp = ctypes.c_void_p


class KsmmTile(ctypes.Structure):
    _fields_ = [("algo", c_int), ("variant", c_int), ("tile_m", c_int), ("tile_n", c_int),
                ("tile_k", c_int), ("tile_d", c_int), ("threads", c_int), ("lds_bytes", c_int),
                ("grid", c_i64)]

    def as_dict(self):
        return {k: getattr(self, k) for k, _ in self._fields_}


class KsmmFactorDesc(ctypes.Structure):
    _fields_ = [("w", c_vp), ("a", c_int), ("b", c_int), ("c", c_int), ("d", c_int),
                ("w_dtype", c_int), ("scale", ctypes.c_float)]


class KsmmEpilogue(ctypes.Structure):
    _fields_ = [("bias", c_vp), ("act", c_int)]


# name -> (restype, argtypes); every symbol include/ksmm_hip.h declares
SIGNATURES = {
    "ksmm_version": (c_int, []),
    "ksmm_strerror": (ctypes.c_char_p, [c_int]),
    "ksmm_validate": (c_int, [c_i64, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int]),
    "ksmm_query_tile": (c_int, [c_i64, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                ctypes.POINTER(KsmmTile)]),
    "ksmm_query_tile_variant": (c_int, [c_i64, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                        c_int, ctypes.POINTER(KsmmTile)]),
    "ksmm_tuned_count": (c_int, []),
    "ksmm_tuned_row": (c_int, [c_int, ctypes.POINTER(c_int * 10)]),
    "ksmm_variant_id": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int, ctypes.POINTER(ctypes.c_uint32),
                                ctypes.POINTER(c_int)]),
    "ksmm_variant_from_id": (c_int, [c_int, ctypes.c_uint32, c_int, c_int, c_int, c_int, c_int,
                                     ctypes.POINTER(c_int)]),
    "ksmm_factor_forward": (c_int, [c_vp, c_vp, c_vp, c_i64, c_int, c_int, c_int, c_int, c_int, c_int,
                                    c_int, c_int, ctypes.c_float, c_vp]),
    "ksmm_factor_forward_algo": (c_int, [c_vp, c_vp, c_vp, c_i64, c_int, c_int, c_int, c_int, c_int,
                                         c_int, c_int, c_int, ctypes.c_float, c_int, c_int, c_vp]),
    "ksmm_factor_workspace": (c_i64, [c_i64, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int]),
    "ksmm_factor_forward_ws": (c_int, [c_vp, c_vp, c_vp, c_i64, c_int, c_int, c_int, c_int, c_int, c_int,
                                       c_int, c_int, ctypes.c_float, c_vp, c_i64, c_vp]),
    "ksmm_chain_workspace": (c_i64, [ctypes.POINTER(KsmmFactorDesc), c_int, c_i64, c_int]),
    "ksmm_chain_workspace_layout": (c_i64, [ctypes.POINTER(KsmmFactorDesc), c_int, c_i64, c_int, c_int,
                                            c_int]),
    "ksmm_chain_forward": (c_int, [ctypes.POINTER(KsmmFactorDesc), c_int, c_vp, c_vp, c_vp, c_i64,
                                   c_i64, c_int, c_int, c_int, c_int, c_vp]),
    "ksmm_factor_forward_ep": (c_int, [c_vp, c_vp, c_vp, c_i64, c_int, c_int, c_int, c_int, c_int, c_int,
                                       c_int, c_int, ctypes.c_float, ctypes.POINTER(KsmmEpilogue), c_vp, c_i64,
                                       c_vp]),
    "ksmm_chain_forward_ep": (c_int, [ctypes.POINTER(KsmmFactorDesc), c_int, c_vp, c_vp, c_vp, c_i64,
                                      c_i64, c_int, c_int, c_int, c_int, ctypes.POINTER(KsmmEpilogue), c_vp]),
    "ksmm_factor_backward_workspace": (c_i64, [c_i64, c_int, c_int, c_int, c_int, c_int, c_int]),
    "ksmm_factor_backward_input": (c_int, [c_vp, c_vp, c_vp, c_i64, c_int, c_int, c_int, c_int, c_int, c_int,
                                           ctypes.c_float, c_vp, c_i64, c_vp]),
    "ksmm_factor_backward_weight": (c_int, [c_vp, c_vp, c_vp, c_i64, c_int, c_int, c_int, c_int, c_int, c_int,
                                            ctypes.c_float, c_vp, c_i64, c_vp]),
    "ksmm_static_scratch_bytes": (c_i64, []),
    "ksmm_chain_forward_static": (c_int, [ctypes.POINTER(KsmmFactorDesc), c_int, c_vp, c_vp, c_i64, c_int,
                                          c_int, c_int, c_int, ctypes.POINTER(KsmmEpilogue), c_vp]),
}

_lib = None


class KsmmError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("ksmm: %s (status %d)" % (message, status))
        self.status = status


def load():
    """Load the shared library (once) and declare the signatures."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libksmm_hip.so is not built (%s missing): run `python -m ksmm_amd.build`. "
            "algo='kernel' has no fallback." % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if lib.ksmm_version() != ABI_VERSION:
        raise ImportError("libksmm_hip.so has ABI version %d, expected %d: rebuild it with "
                          "`python -m ksmm_amd.build`" % (lib.ksmm_version(), ABI_VERSION))
    _lib = lib
    return lib


def strerror(status):
    return load().ksmm_strerror(status).decode()


def check(status):
    if status != 0:
        raise KsmmError(status, strerror(status))
