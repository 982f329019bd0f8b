"""ctypes binding over ``libpenc_probes.so`` (``include/penc_probes.h``): the memory-system probes the
benchmark prices the encoding's traffic against.  Measurement aids only; the encoding never loads them."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpenc_probes.so")
_lib = None

_p = ctypes.c_void_p
_SIGNATURES = {
    "penc_probe_copy": (ctypes.c_int, [_p, _p, ctypes.c_int64, _p]),
    "penc_probe_read": (ctypes.c_int, [_p, ctypes.c_int64, _p, _p]),
    "penc_probe_gather": (ctypes.c_int, [_p, _p, ctypes.c_int64, ctypes.c_int, _p, _p]),
    "penc_probe_gather_variant": (ctypes.c_int, [_p, ctypes.c_int64, _p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                ctypes.c_int, _p, _p]),
    "penc_probe_scatter": (ctypes.c_int, [_p, _p, ctypes.c_int64, ctypes.c_int, _p]),
}
EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def lib():
    """Loads the probe library once; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m permutohedral_encoding_amd.build`")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib
