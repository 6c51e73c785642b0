"""ctypes access to oracle/libnorm_ref.so, the C restatement of the reference
arithmetic (TEST INFRASTRUCTURE / CPU BASELINE ONLY).  float32 numpy arrays in
and out."""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnorm_ref.so")
_lib = None

_P = ctypes.c_void_p
_I = ctypes.c_int64
_F = ctypes.c_float
_i = ctypes.c_int


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} missing: run `make -C {_HERE}`")
        L = ctypes.CDLL(LIB_PATH)
        L.nr_num_threads.restype = _i
        L.nr_set_num_threads.argtypes = [_i]
        L.nr_set_num_threads.restype = None
        L.nr_bn_forward_global.argtypes = [_P] * 6 + [_I] * 3 + [_F]
        L.nr_bn_forward_batch.argtypes = [_P] * 8 + [_I] * 3 + [_F, _F]
        L.nr_bn_backward_batch.argtypes = [_P] * 10 + [_I] * 3 + [_F]
        L.nr_ln_forward.argtypes = [_P] * 6 + [_I] * 2 + [_F]
        L.nr_ln_backward.argtypes = [_P] * 10 + [_I] * 2 + [_F]
        L.nr_gn_forward.argtypes = [_P] * 6 + [_I] * 4 + [_F]
        L.nr_gn_backward.argtypes = [_P] * 11 + [_I] * 4 + [_F]
        L.nr_in_forward.argtypes = [_P] * 6 + [_I] * 3 + [_i, _i, _F]
        L.nr_in_backward.argtypes = [_P] * 11 + [_I] * 3 + [_i, _i, _F]
        for name in ("nr_bn_forward_global", "nr_bn_forward_batch", "nr_bn_backward_batch",
                     "nr_ln_forward", "nr_ln_backward", "nr_gn_forward", "nr_gn_backward",
                     "nr_in_forward", "nr_in_backward"):
            getattr(L, name).restype = None
        _lib = L
    return _lib


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return None if a is None else a.ctypes.data_as(_P)


def bn_forward_global(x, beta, gamma, rmean, rvar, size0, c, size2, eps=1e-5):
    x, beta, gamma, rmean, rvar = map(_f32, (x, beta, gamma, rmean, rvar))
    y = np.empty_like(x)
    lib().nr_bn_forward_global(_p(x), _p(beta), _p(gamma), _p(rmean), _p(rvar), _p(y), size0, c,
                               size2, eps)
    return y


def bn_forward_batch(x, beta, gamma, rmean, rvar, size0, c, size2, decay=0.9, eps=1e-5):
    """rmean/rvar (float32 arrays or None) are updated in place."""
    x, beta, gamma = map(_f32, (x, beta, gamma))
    y = np.empty_like(x)
    mean = np.empty(c, np.float32)
    var = np.empty(c, np.float32)
    lib().nr_bn_forward_batch(_p(x), _p(beta), _p(gamma), _p(rmean), _p(rvar), _p(y), _p(mean),
                              _p(var), size0, c, size2, decay, eps)
    return y, mean, var


def bn_backward_batch(x, dy, gamma, mean, var, size0, c, size2, eps=1e-5, dmean=None, dvar=None):
    x, dy, gamma, mean, var, dmean, dvar = map(_f32, (x, dy, gamma, mean, var, dmean, dvar))
    dx = np.empty_like(x)
    dg = np.empty(c, np.float32)
    db = np.empty(c, np.float32)
    lib().nr_bn_backward_batch(_p(x), _p(dy), _p(gamma), _p(mean), _p(var), _p(dmean), _p(dvar),
                               _p(dx), _p(dg), _p(db), size0, c, size2, eps)
    return dx, dg, db


def ln_forward(x, beta, gamma, outer, eps=1e-5):
    x, beta, gamma = map(_f32, (x, beta, gamma))
    r = x.size // outer
    y = np.empty_like(x)
    mean = np.empty(outer, np.float32)
    var = np.empty(outer, np.float32)
    lib().nr_ln_forward(_p(x), _p(beta), _p(gamma), _p(y), _p(mean), _p(var), outer, r, eps)
    return y, mean, var


def ln_backward(x, dy, gamma, mean, var, outer, eps=1e-5, dmean=None, dvar=None):
    x, dy, gamma, mean, var, dmean, dvar = map(_f32, (x, dy, gamma, mean, var, dmean, dvar))
    r = x.size // outer
    dx = np.empty_like(x)
    dg = np.empty(r, np.float32)
    db = np.empty(r, np.float32)
    lib().nr_ln_backward(_p(x), _p(dy), _p(gamma), _p(mean), _p(var), _p(dmean), _p(dvar), _p(dx),
                         _p(dg), _p(db), outer, r, eps)
    return dx, dg, db


def gn_forward(x, beta, gamma, n, c, s, groups, eps=1e-5):
    x, beta, gamma = map(_f32, (x, beta, gamma))
    y = np.empty_like(x)
    mean = np.empty(n * groups, np.float32)
    var = np.empty(n * groups, np.float32)
    lib().nr_gn_forward(_p(x), _p(beta), _p(gamma), _p(y), _p(mean), _p(var), n, c, s, groups, eps)
    return y, mean, var


def gn_backward(x, dy, gamma, mean, var, n, c, s, groups, eps=1e-5, dmean=None, dvar=None):
    x, dy, gamma, mean, var, dmean, dvar = map(_f32, (x, dy, gamma, mean, var, dmean, dvar))
    dx = np.empty_like(x)
    dg = np.empty(c, np.float32)
    db = np.empty(c, np.float32)
    scratch = np.empty(2 * n * c, np.float64)
    lib().nr_gn_backward(_p(x), _p(dy), _p(gamma), _p(mean), _p(var), _p(dmean), _p(dvar), _p(dx),
                         _p(dg), _p(db), _p(scratch), n, c, s, groups, eps)
    return dx, dg, db


def in_forward(x, beta, gamma, n, c, s, bc_gamma=True, bc_beta=True, eps=1e-5):
    x, beta, gamma = map(_f32, (x, beta, gamma))
    y = np.empty_like(x)
    mean = np.empty(n * c, np.float32)
    var = np.empty(n * c, np.float32)
    lib().nr_in_forward(_p(x), _p(beta), _p(gamma), _p(y), _p(mean), _p(var), n, c, s,
                        int(bc_gamma), int(bc_beta), eps)
    return y, mean, var


def in_backward(x, dy, gamma, mean, var, n, c, s, bc_gamma=True, bc_beta=True, eps=1e-5,
                dmean=None, dvar=None):
    x, dy, gamma, mean, var, dmean, dvar = map(_f32, (x, dy, gamma, mean, var, dmean, dvar))
    dx = np.empty_like(x)
    dg = np.empty(c if bc_gamma else n * c, np.float32)
    db = np.empty(c if bc_beta else n * c, np.float32)
    scratch = np.empty(2 * n * c, np.float64)
    lib().nr_in_backward(_p(x), _p(dy), _p(gamma), _p(mean), _p(var), _p(dmean), _p(dvar), _p(dx),
                         _p(dg), _p(db), _p(scratch), n, c, s, int(bc_gamma), int(bc_beta), eps)
    return dx, dg, db
