"""Randomly drawn shapes (fixed seeds) for every family, layout and dtype: the
HIP path through the C-ABI against the float64 oracle.

The targeted shape lists of the other test files aim at one kernel layout each;
the launcher picks among a few dozen layouts by thresholds on the shape, and
this file walks that decision space without aiming: log-uniform sizes, odd and
even extents, few and many channels, groups of every divisor.  Reductions of
fewer than 6 elements are left out (their variance is too ill-conditioned for
the float32 tolerance; the targeted lists hold such shapes with their own
bounds)."""
import numpy as np
import pytest
import torch

from _util import assert_close, dtype_name, load_package, rounded, to_dev, to_np
from oracle import norm_ref as R

pytestmark = pytest.mark.gpu
K = load_package()
DTYPES = [torch.float32, torch.float16]
MAX_ELEMS = 1 << 19  # keeps the float64 oracle at milliseconds per case


def f32(a):
    return np.asarray(a, np.float32).astype(np.float64)


def log_int(rng, lo, hi):
    return int(round(float(np.exp(rng.uniform(np.log(lo), np.log(hi))))))


def draw_ncs(rng):
    """(n, c, spatial tuple) with n*c*prod(spatial) <= MAX_ELEMS."""
    while True:
        n = log_int(rng, 1, 64)
        c = log_int(rng, 1, 2048)
        nd = int(rng.integers(1, 3))
        sp = tuple(log_int(rng, 1, 96) for _ in range(nd))
        if n * c * int(np.prod(sp)) <= MAX_ELEMS:
            return n, c, sp


def divisors(c):
    return [d for d in range(1, c + 1) if c % d == 0]


# ---------------------------------------------------------------- BatchNormalization
@pytest.mark.parametrize("seed", range(40))
@pytest.mark.parametrize("dtype", DTYPES)
def test_random_bn(seed, dtype):
    rng = np.random.default_rng(1000 + seed)
    while True:
        n, c, sp = draw_ncs(rng)
        if n * int(np.prod(sp)) >= 6:
            break
    channel_last = bool(rng.integers(0, 2))
    shape = (n,) + sp + (c,) if channel_last else (n, c) + sp
    axis = len(shape) - 1 if channel_last else 1
    dn = dtype_name(dtype)
    x = rounded(rng.standard_normal(shape) * 2.0 + 1.0, dtype)
    dy = rounded(rng.standard_normal(shape), dtype)
    g, b = f32(rng.uniform(0.5, 1.5, c)), f32(rng.standard_normal(c) * 0.1)
    rm, rv = f32(rng.standard_normal(c) * 0.1), f32(rng.uniform(0.5, 2, c))
    y_r, m_r, v_r, rm_r, rv_r = R.bn_forward_batch(x, b, g, rm, rv, axis, 0.9, 1e-5)
    dx_r, dg_r, db_r = R.bn_backward_batch(x, dy, g, m_r, v_r, axis, 1e-5)
    xd, dyd, gd, bd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(b)
    rmd, rvd = to_dev(rm), to_dev(rv)
    y, m, v = K.bn_forward_batch(xd, bd, gd, rmd, rvd, axis, 0.9, 1e-5)
    what = f"shape {shape} axis {axis}"
    assert_close(to_np(y), y_r, dn, "y", "y " + what)
    assert_close(to_np(m), m_r, dn, "stat", "mean " + what)
    assert_close(to_np(v), v_r, dn, "stat", "var " + what)
    assert_close(to_np(rmd), rm_r, dn, "stat", "running_mean " + what)
    assert_close(to_np(rvd), rv_r, dn, "stat", "running_var " + what)
    dx, dg, db = K.bn_backward(xd, dyd, gd, m, v, axis, 1e-5)
    assert_close(to_np(dx), dx_r, dn, "grad", "dx " + what)
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma " + what)
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta " + what)
    # inference forward on the same tensor
    yi = K.bn_forward_global(xd, bd, gd, to_dev(rm), to_dev(rv), axis, 1e-5)
    assert_close(to_np(yi), R.bn_forward_global(x, b, g, rm, rv, axis, 1e-5), dn, "y",
                 "inference y " + what)


# ---------------------------------------------------------------- LayerNormalization
@pytest.mark.parametrize("seed", range(40))
@pytest.mark.parametrize("dtype", DTYPES)
def test_random_ln(seed, dtype):
    rng = np.random.default_rng(2000 + seed)
    while True:
        outer, Rr = log_int(rng, 1, 20000), log_int(rng, 6, 100000)
        if outer * Rr <= MAX_ELEMS:
            break
    dn = dtype_name(dtype)
    x = rounded(rng.standard_normal((outer, Rr)) + rng.uniform(-3, 3, (outer, 1)), dtype)
    dy = rounded(rng.standard_normal((outer, Rr)), dtype)
    g, b = f32(rng.standard_normal(Rr) * 0.1 + 1), f32(rng.standard_normal(Rr) * 0.1)
    y_r, m_r, v_r = R.ln_forward(x, b, g, outer, 1e-5)
    dx_r, dg_r, db_r = R.ln_backward(x, dy, g, m_r, v_r, outer, 1e-5)
    xd, dyd, gd, bd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(b)
    y, m, v = K.ln_forward(xd, bd, gd, outer, 1e-5)
    what = f"rows {outer} x {Rr}"
    assert_close(to_np(m), m_r, dn, "stat", "mean " + what)
    assert_close(to_np(v), v_r, dn, "stat", "var " + what)
    assert_close(to_np(y), y_r, dn, "y", "y " + what)
    dx, dg, db = K.ln_backward(xd, dyd, gd, m, v, outer, 1e-5)
    assert_close(to_np(dx), dx_r, dn, "grad", "dx " + what)
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma " + what)
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta " + what)


# ------------------------------------------- GroupNormalization / InstanceNormalization
@pytest.mark.parametrize("seed", range(50))
@pytest.mark.parametrize("dtype", DTYPES)
def test_random_gn_in(seed, dtype):
    rng = np.random.default_rng(3000 + seed)
    instance = seed % 3 == 0
    while True:
        n, c, sp = draw_ncs(rng)
        groups = c if instance else int(rng.choice(divisors(c)))
        if (c // groups) * int(np.prod(sp)) >= 6:
            break
    channel_last = bool(rng.integers(0, 2))
    dn = dtype_name(dtype)
    cf_shape = (n, c) + sp
    x = rounded(rng.standard_normal(cf_shape) * 1.5, dtype)      # channel-first view
    dy = rounded(rng.standard_normal(cf_shape), dtype)
    g, b = f32(rng.uniform(0.5, 1.5, c)), f32(rng.standard_normal(c) * 0.1)
    if instance:
        y_r, m_r, v_r = R.in_forward(x, b, g, n, c, 1e-5)
        dx_r, dg_r, db_r = R.in_backward(x, dy, g, m_r, v_r, n, c, 1e-5)
    else:
        y_r, m_r, v_r = R.gn_forward(x, b, g, n, c, groups, 1e-5)
        dx_r, dg_r, db_r = R.gn_backward(x, dy, g, m_r, v_r, n, c, groups, 1e-5)

    def dev(a):
        if channel_last:
            a = np.ascontiguousarray(np.moveaxis(a, 1, -1))
        return to_dev(a, dtype)

    def host(t):
        a = to_np(t)
        return np.moveaxis(a, -1, 1) if channel_last else a

    xd, dyd, gd, bd = dev(x), dev(dy), to_dev(g), to_dev(b)
    what = f"{'IN' if instance else 'GN'} n {n} c {c} spatial {sp} groups {groups} " \
           f"{'channel-last' if channel_last else 'channel-first'}"
    if instance:
        y, m, v = K.in_forward(xd, bd, gd, 1e-5, channel_last=channel_last)
    else:
        y, m, v = K.gn_forward(xd, bd, gd, groups, 1e-5, channel_last=channel_last)
    assert_close(to_np(m).reshape(-1), np.asarray(m_r).reshape(-1), dn, "stat", "mean " + what)
    assert_close(to_np(v).reshape(-1), np.asarray(v_r).reshape(-1), dn, "stat", "var " + what)
    assert_close(host(y), y_r, dn, "y", "y " + what)
    if instance:
        dx, dg, db = K.in_backward(xd, dyd, gd, m, v, 1e-5, channel_last=channel_last)
    else:
        dx, dg, db = K.gn_backward(xd, dyd, gd, m, v, groups, 1e-5, channel_last=channel_last)
    assert_close(host(dx), dx_r, dn, "grad", "dx " + what)
    assert_close(to_np(dg).reshape(-1), np.asarray(dg_r).reshape(-1), dn, "pgrad", "dgamma " + what)
    assert_close(to_np(db).reshape(-1), np.asarray(db_r).reshape(-1), dn, "pgrad", "dbeta " + what)
