"""ctypes binding of libksmm_bench.so: the measurement aids bench.py times beside the kernels
(matrix-core rate on register operands, tile-at-a-time copy, streaming copy; declared in
ksmm_amd/csrc/ksmm_probe.h).  Built by ``python -m ksmm_amd.build`` next to libksmm_hip.so; not
part of the drop-in ABI."""
import ctypes
import os

from ._lib import c_i64, c_int, c_vp

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libksmm_bench.so")

SIGNATURES = {
    "ksbench_mfma_probe_bytes": (c_i64, []),
    "ksbench_mfma_probe": (c_int, [c_int, c_int, c_int, c_vp, c_i64, ctypes.POINTER(ctypes.c_double), c_vp]),
    "ksbench_tilecopy_probe": (c_int, [c_vp, c_vp, c_i64, c_int, c_int, c_int, c_int, c_vp]),
    "ksbench_stream_copy": (c_int, [c_vp, c_vp, c_i64, c_int, c_vp]),
}

_lib = None


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError("libksmm_bench.so is not built (%s missing): run `python -m ksmm_amd.build`" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib
