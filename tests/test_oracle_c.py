"""The C restatement (oracle/norm_ref.c, the timed CPU baseline) against the
pinned float64 oracle on seeded inputs."""
import os
import subprocess

import numpy as np
import pytest

from _util import ROOT
from oracle import c_ref as C
from oracle import norm_ref as R


@pytest.fixture(scope="module", autouse=True)
def built():
    if not os.path.exists(C.LIB_PATH):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])


def close(a, b, tol=2e-6):
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    scale = max(1.0, float(np.sqrt(np.mean(b * b))))
    assert np.abs(a - b).max() <= tol * scale + tol * np.abs(b).max()


def f32(a):
    return np.asarray(a, np.float32)


@pytest.mark.parametrize("shape,axis", [((4, 3, 5, 2), 1), ((6, 7), 1), ((3, 4, 5), 2), ((9, 2, 17), 1)])
def test_bn(shape, axis):
    rng = np.random.default_rng(0)
    c = shape[axis]
    s0 = int(np.prod(shape[:axis]))
    s2 = int(np.prod(shape[axis + 1:]))
    x = f32(rng.standard_normal(shape) * 2 + 1)
    dy = f32(rng.standard_normal(shape))
    g, b = f32(rng.uniform(0.5, 1.5, c)), f32(rng.standard_normal(c))
    rm, rv = f32(rng.standard_normal(c)), f32(rng.uniform(0.5, 2, c))
    dm, dv = f32(rng.standard_normal(c)), f32(rng.standard_normal(c))
    close(C.bn_forward_global(x, b, g, rm, rv, s0, c, s2), R.bn_forward_global(x, b, g, rm, rv, axis))
    y_r, m_r, v_r, rm_r, rv_r = R.bn_forward_batch(x, b, g, rm, rv, axis, 0.9, 1e-5)
    rm_c, rv_c = rm.copy(), rv.copy()
    y, m, v = C.bn_forward_batch(x, b, g, rm_c, rv_c, s0, c, s2, 0.9, 1e-5)
    close(y, y_r); close(m, m_r); close(v, v_r); close(rm_c, rm_r); close(rv_c, rv_r)
    dx_r, dg_r, db_r = R.bn_backward_batch(x, dy, g, m, v, axis, 1e-5, dm, dv)
    dx, dg, db = C.bn_backward_batch(x, dy, g, m, v, s0, c, s2, 1e-5, dm, dv)
    close(dx, dx_r); close(dg, dg_r); close(db, db_r)


@pytest.mark.parametrize("outer,Rr", [(4, 6), (5, 33), (1, 17), (7, 1)])
def test_ln(outer, Rr):
    rng = np.random.default_rng(1)
    x, dy = f32(rng.standard_normal((outer, Rr)) + 2), f32(rng.standard_normal((outer, Rr)))
    g, b = f32(rng.uniform(0.5, 1.5, Rr)), f32(rng.standard_normal(Rr))
    dm, dv = f32(rng.standard_normal(outer)), f32(rng.standard_normal(outer))
    y_r, m_r, v_r = R.ln_forward(x, b, g, outer, 1e-5)
    y, m, v = C.ln_forward(x, b, g, outer, 1e-5)
    close(y, y_r); close(m, m_r); close(v, v_r)
    dx_r, dg_r, db_r = R.ln_backward(x, dy, g, m, v, outer, 1e-5, dm, dv)
    dx, dg, db = C.ln_backward(x, dy, g, m, v, outer, 1e-5, dm, dv)
    close(dx, dx_r, 1e-5); close(dg, dg_r); close(db, db_r)


@pytest.mark.parametrize("n,c,s,groups", [(2, 8, 9, 4), (3, 6, 5, 2), (2, 6, 4, 6), (1, 4, 1, 2)])
def test_gn(n, c, s, groups):
    rng = np.random.default_rng(2)
    x, dy = f32(rng.standard_normal((n, c, s)) * 1.5), f32(rng.standard_normal((n, c, s)))
    g, b = f32(rng.uniform(0.5, 1.5, c)), f32(rng.standard_normal(c))
    dm, dv = f32(rng.standard_normal(n * groups)), f32(rng.standard_normal(n * groups))
    y_r, m_r, v_r = R.gn_forward(x, b, g, n, c, groups, 1e-5)
    y, m, v = C.gn_forward(x, b, g, n, c, s, groups, 1e-5)
    close(y, y_r); close(m, m_r); close(v, v_r)
    dx_r, dg_r, db_r = R.gn_backward(x, dy, g, m, v, n, c, groups, 1e-5, dm, dv)
    dx, dg, db = C.gn_backward(x, dy, g, m, v, n, c, s, groups, 1e-5, dm, dv)
    close(dx, dx_r, 1e-5); close(dg, dg_r); close(db, db_r)


@pytest.mark.parametrize("n,c,s", [(2, 3, 16), (3, 5, 7)])
@pytest.mark.parametrize("bcg,bcb", [(True, True), (False, False), (True, False)])
def test_in(n, c, s, bcg, bcb):
    rng = np.random.default_rng(3)
    x, dy = f32(rng.standard_normal((n, c, s)) * 1.5), f32(rng.standard_normal((n, c, s)))
    g = f32(rng.uniform(0.5, 1.5, c if bcg else n * c))
    b = f32(rng.standard_normal(c if bcb else n * c))
    dm, dv = f32(rng.standard_normal(n * c)), f32(rng.standard_normal(n * c))
    g_full = np.tile(g, n) if bcg else g
    b_full = np.tile(b, n) if bcb else b
    y_r, m_r, v_r = R.in_forward(x, b_full, g_full, n, c, 1e-5)
    y, m, v = C.in_forward(x, b, g, n, c, s, bcg, bcb, 1e-5)
    close(y, y_r); close(m, m_r); close(v, v_r)
    dx_r, dg_r, db_r = R.in_backward(x, dy, g, m, v, n, c, 1e-5, dm, dv, bc_gamma=bcg, bc_beta=bcb)
    dx, dg, db = C.in_backward(x, dy, g, m, v, n, c, s, bcg, bcb, 1e-5, dm, dv)
    close(dx, dx_r, 1e-5); close(dg, dg_r); close(db, db_r)
