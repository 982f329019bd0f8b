"""ctypes binding over the CPU oracle library (test infrastructure; see ``penc_oracle.cpp``).

All functions take and return NumPy arrays.  Layouts follow the reference's kernels:
positions ``(N, D)``, table ``(L, C, F)``, scale factors / shifts ``(L, D)``, window ``(L,)``,
sliced values and their gradients ``(L [+extra], F, N)``, table gradients ``(L, C, F)``,
position gradients ``(N, D)``.  F, the number of features per level, is read off the table's or the
gradient's shape (the reference supports F = 2 only).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# PENC_ORACLE_LIB lets a mutated build be swapped in when checking that the pinning tests discriminate
_LIB_PATH = os.environ.get("PENC_ORACLE_LIB", os.path.join(_HERE, "libpenc_oracle.so"))
_lib = None


def build(force=False):
    """Compile the oracle with the Makefile next to this file."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _f(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def _check(rc, what):
    if rc != 0:
        raise ValueError(f"oracle {what} failed with status {rc}")


def num_threads():
    return int(lib().penc_oracle_num_threads())


def extra_levels(pos_dim, concat_points, nr_feat=2):
    return (pos_dim + nr_feat - 1) // nr_feat if concat_points else 0


def hash_key(key):
    key = _f(key, np.int32)
    out = ctypes.c_uint32(0)
    _check(lib().penc_oracle_hash(int(key.size), _p(key), ctypes.byref(out)), "hash")
    return int(out.value)


def slot(key, capacity):
    key = _f(key, np.int32)
    out = ctypes.c_int(0)
    _check(lib().penc_oracle_slot(int(key.size), _p(key), int(capacity), ctypes.byref(out)), "slot")
    return int(out.value)


def scale_factors(pos_dim, sigmas):
    sigmas = _f(sigmas, np.float32)
    sf = np.empty((sigmas.size, pos_dim), np.float32)
    _check(lib().penc_oracle_scale_factors(int(pos_dim), int(sigmas.size), _p(sigmas), _p(sf)), "scale_factors")
    return sf


def _dims(pos, shift):
    n, d = pos.shape
    l = shift.shape[0]
    assert shift.shape == (l, d)
    return ctypes.c_int64(n), int(d), int(l)


def simplex(pos, sf, shift, capacity, dtype=np.float32, with_keys=False):
    """Per (level, point): elevated (L,N,D+1), rem0, rank, bary (first D+1 weights), slot, [keys (L,N,D+1,D+1)]."""
    pos, sf, shift = _f(pos, dtype), _f(sf, dtype), _f(shift, dtype)
    n, d, l = _dims(pos, shift)
    shp = (l, pos.shape[0], d + 1)
    out = dict(elevated=np.empty(shp, dtype), rem0=np.empty(shp, np.int32), rank=np.empty(shp, np.int32),
               bary=np.empty(shp, dtype), slot=np.empty(shp, np.int32))
    keys = np.empty(shp + (d + 1,), np.int32) if with_keys else None
    fn = lib().penc_oracle_simplex if dtype == np.float32 else lib().penc_oracle_simplex_f64
    _check(fn(d, n, l, int(capacity), _p(pos), _p(sf), _p(shift), _p(out["elevated"]), _p(out["rem0"]),
              _p(out["rank"]), _p(out["bary"]), _p(out["slot"]), _p(keys)), "simplex")
    if with_keys:
        out["keys"] = keys
    return out


def forward(pos, table, sf, shift, window, concat_points=False, points_scaling=1.0, dtype=np.float32):
    pos, table, sf, shift, window = (_f(a, dtype) for a in (pos, table, sf, shift, window))
    n, d, l = _dims(pos, shift)
    c, f = table.shape[1], table.shape[2]
    assert table.shape == (l, c, f) and window.shape == (l,)
    out = np.empty((l + extra_levels(d, concat_points, f), f, pos.shape[0]), dtype)
    if dtype == np.float32:
        rc = lib().penc_oracle_forward(d, n, l, c, f, _p(pos), _p(table), _p(sf), _p(shift), _p(window), _p(out),
                                       int(bool(concat_points)), ctypes.c_float(points_scaling))
    else:
        rc = lib().penc_oracle_forward_f64(d, n, l, c, f, _p(pos), _p(table), _p(sf), _p(shift), _p(window), _p(out),
                                           int(bool(concat_points)), ctypes.c_double(points_scaling))
    _check(rc, "forward")
    return out


def backward_table(pos, sf, shift, window, grad, capacity, dtype=np.float32, want32=True, want64=True, want_abs=False):
    """Returns dict(grad32=(L,C,2) fp32 omp-atomic sum, grad64=fp64 sum, abs64=fp64 sum of |terms|)."""
    pos, sf, shift, window, grad = (_f(a, dtype) for a in (pos, sf, shift, window, grad))
    n, d, l = _dims(pos, shift)
    c, f = int(capacity), grad.shape[1]
    assert grad.shape[0] >= l and grad.shape[1:] == (f, pos.shape[0])
    if dtype == np.float64:
        g = np.zeros((l, c, f), np.float64)
        _check(lib().penc_oracle_backward_table_f64(d, n, l, c, f, _p(pos), _p(sf), _p(shift), _p(window), _p(grad), _p(g)),
               "backward_table_f64")
        return dict(grad64=g)
    g32 = np.zeros((l, c, f), np.float32) if want32 else None
    g64 = np.zeros((l, c, f), np.float64) if want64 else None
    a64 = np.zeros((l, c, f), np.float64) if want_abs else None
    _check(lib().penc_oracle_backward_table(d, n, l, c, f, _p(pos), _p(sf), _p(shift), _p(window), _p(grad),
                                            _p(g32), _p(g64), _p(a64)), "backward_table")
    return dict(grad32=g32, grad64=g64, abs64=a64)


def backward_pos(pos, table, sf, shift, window, grad, dtype=np.float32):
    """Returns dict(grad32=(N,D), grad64=(N,D) fp64-accumulated over levels, abs64=(N,D) the same chain
    with every term replaced by its magnitude: the scale the rounding error of grad32 is relative to)."""
    pos, table, sf, shift, window, grad = (_f(a, dtype) for a in (pos, table, sf, shift, window, grad))
    n, d, l = _dims(pos, shift)
    c, f = table.shape[1], table.shape[2]
    if dtype == np.float64:
        g = np.empty(pos.shape, np.float64)
        _check(lib().penc_oracle_backward_pos_f64(d, n, l, c, f, _p(pos), _p(table), _p(sf), _p(shift), _p(window),
                                                  _p(grad), _p(g)), "backward_pos_f64")
        return dict(grad64=g)
    g32 = np.empty(pos.shape, np.float32)
    g64 = np.empty(pos.shape, np.float64)
    a64 = np.empty(pos.shape, np.float64)
    _check(lib().penc_oracle_backward_pos(d, n, l, c, f, _p(pos), _p(table), _p(sf), _p(shift), _p(window), _p(grad),
                                          _p(g32), _p(g64), _p(a64)), "backward_pos")
    return dict(grad32=g32, grad64=g64, abs64=a64)


def double_backward(pos, table, sf, shift, window, double_pos_grad, grad, concat_points=False, dtype=np.float32,
                    want32=True, want64=True, want_abs=False):
    """Returns dict(grad32/grad64/abs64 = table gradient (L,C,2), ggs = (L+extra,2,N), and with want_abs
    ggs_abs64 = the grad-of-grad chain with every term replaced by its magnitude)."""
    pos, table, sf, shift, window, q, grad = (_f(a, dtype) for a in (pos, table, sf, shift, window, double_pos_grad, grad))
    n, d, l = _dims(pos, shift)
    c, f = table.shape[1], table.shape[2]
    assert q.shape == pos.shape
    ggs = np.empty((l + extra_levels(d, concat_points, f), f, pos.shape[0]), dtype)
    if dtype == np.float64:
        g = np.zeros((l, c, f), np.float64)
        _check(lib().penc_oracle_double_backward_f64(d, n, l, c, f, _p(pos), _p(table), _p(sf), _p(shift), _p(window),
                                                     _p(q), _p(grad), _p(g), _p(ggs), int(bool(concat_points))),
               "double_backward_f64")
        return dict(grad64=g, ggs=ggs)
    g32 = np.zeros((l, c, f), np.float32) if want32 else None
    g64 = np.zeros((l, c, f), np.float64) if want64 else None
    a64 = np.zeros((l, c, f), np.float64) if want_abs else None
    ga64 = np.empty(ggs.shape, np.float64) if want_abs else None
    _check(lib().penc_oracle_double_backward(d, n, l, c, f, _p(pos), _p(table), _p(sf), _p(shift), _p(window), _p(q),
                                             _p(grad), _p(g32), _p(g64), _p(a64), _p(ggs), _p(ga64),
                                             int(bool(concat_points))),
           "double_backward")
    return dict(grad32=g32, grad64=g64, abs64=a64, ggs=ggs, ggs_abs64=ga64)
