"""Randomly drawn calls with randomly drawn flags (fixed seeds): every family,
both layouts and dtypes, tensors of 20 KB - 24 MB, with or without gamma / beta,
with or without the gradients of the statistics (the three-output form), each
of dx / dgamma / dbeta wanted or not (propagate_down) and accumulated or
overwritten - against the oracle, the outputs that are not wanted left as they
were.  (Reduction units of at least six elements: a unit of one or two
elements has no variance to speak of, and 1 / sqrt(eps) = 316 then scales the
rounding of x * a + b, here as in the reference's kernels.)"""
import numpy as np
import pytest
import torch

from _util import assert_close, dtype_name, load_package, rounded, to_dev, to_np
from oracle import norm_ref as R

pytestmark = pytest.mark.gpu
K = load_package()
F16, F32 = torch.float16, torch.float32
LAST_CASE = {}  # what the failing case was, for the assertion message


def f32(a):
    return np.asarray(a, np.float32).astype(np.float64)


def divisors(c):
    return [d for d in range(1, c + 1) if c % d == 0]


def logi(rng, lo, hi):
    return int(np.exp(rng.uniform(np.log(lo), np.log(hi))))


def one_case(rng):
    kind = str(rng.choice(["bn", "ln", "gn", "in"]))
    dt = F16 if rng.integers(0, 2) else F32
    dn = dtype_name(dt)
    esz = 2 if dt == F16 else 4
    target = logi(rng, 2e4, 24e6) // esz   # elements
    cl = bool(rng.integers(0, 2)) and kind != "ln"
    use_gamma = rng.random() > 0.2
    use_beta = rng.random() > 0.2
    accum = tuple(bool(rng.integers(0, 2)) for _ in range(3))
    need = tuple(bool(rng.random() > 0.25) for _ in range(3))
    if not any(need):
        need = (True, True, True)
    three = rng.random() < 0.4
    desc = LAST_CASE
    desc.clear()
    desc.update(kind=kind, dt=dn, cl=cl, gamma=use_gamma, beta=use_beta, accum=accum, need=need, three=three)
    if kind == "ln":
        Rr = int(rng.choice([logi(rng, 8, 20000), int(rng.choice([64, 256, 1024, 1023, 4096, 8192, 16384]))]))
        outer = max(1, target // Rr)
        desc.update(outer=outer, R=Rr)
        x = rounded(rng.standard_normal((outer, Rr)) + rng.uniform(-3, 3, (outer, 1)), dt)
        dy = rounded(rng.standard_normal((outer, Rr)), dt)
        g = f32(rng.standard_normal(Rr) * 0.1 + 1) if use_gamma else None
        b = f32(rng.standard_normal(Rr) * 0.1) if use_beta else None
        nstat, nparam = outer, Rr
        fwd_r = lambda: R.ln_forward(x, b, g, outer, 1e-5)
        fwd_d = lambda xd, bd, gd: K.ln_forward(xd, bd, gd, outer, 1e-5)
        bwd_r = lambda m, v, dm, dv: R.ln_backward(x, dy, g, m, v, outer, 1e-5, dm, dv)
        bwd_d = lambda xd, dyd, gd, m, v, **kw: K.ln_backward(xd, dyd, gd, m, v, outer, 1e-5, **kw)
        lay = lambda a: a
    else:
        c = int(rng.choice([3, 8, 16, 24, 32, 40, 64, 72, 96, 100, 128, 200, 256, 320, 512, 1024, 2048]))
        h = int(rng.choice([1, 4, 7, 8, 14, 16, 17, 28, 32, 35, 56, 63, 64, 96]))
        w = h if rng.integers(0, 4) else int(rng.integers(1, 80))
        n = max(1, min(128, target // (h * w * c)))
        if h * w < 6:
            h, w = 3, 2 + int(rng.integers(0, 5))
        shape = (n, c, h, w)
        desc.update(shape=shape)
        x = rounded(rng.standard_normal(shape) * 1.5 + rng.uniform(-2, 2, (n, c, 1, 1)), dt)
        dy = rounded(rng.standard_normal(shape), dt)
        g = f32(rng.uniform(0.5, 1.5, c)) if use_gamma else None
        b = f32(rng.standard_normal(c) * 0.1) if use_beta else None
        lay = (lambda a: np.ascontiguousarray(np.moveaxis(a, 1, -1))) if cl else (lambda a: a)
        nparam = c
        if kind == "bn":
            nstat = c
            rm, rv = f32(rng.standard_normal(c) * 0.1), f32(rng.uniform(0.5, 2.0, c))
            axis = 3 if cl else 1
            gg = g if g is not None else np.ones(c)
            bb = b if b is not None else np.zeros(c)
            fwd_r = lambda: R.bn_forward_batch(x, bb, gg, rm, rv, 1, 0.9, 1e-5)[:3]
            def fwd_d(xd, bd, gd):
                return K.bn_forward_batch(xd, bd if bd is not None else to_dev(bb), gd if gd is not None else to_dev(gg), to_dev(rm), to_dev(rv), axis, 0.9, 1e-5)
            bwd_r = lambda m, v, dm, dv: R.bn_backward_batch(x, dy, gg, m, v, 1, 1e-5, dm, dv)
            bwd_d = lambda xd, dyd, gd, m, v, **kw: K.bn_backward(xd, dyd, gd if gd is not None else to_dev(gg), m, v, axis, 1e-5, **kw)
        elif kind == "gn":
            groups = int(rng.choice(divisors(c)))
            desc.update(groups=groups)
            nstat = n * groups
            fwd_r = lambda: R.gn_forward(x, b, g, n, c, groups, 1e-5)
            fwd_d = lambda xd, bd, gd: K.gn_forward(xd, bd, gd, groups, 1e-5, channel_last=cl)
            bwd_r = lambda m, v, dm, dv: R.gn_backward(x, dy, g, m, v, n, c, groups, 1e-5, dm, dv)
            bwd_d = lambda xd, dyd, gd, m, v, **kw: K.gn_backward(xd, dyd, gd, m, v, groups, 1e-5, channel_last=cl, **kw)
        else:
            nstat = n * c
            fwd_r = lambda: R.in_forward(x, b, g, n, c, 1e-5)
            fwd_d = lambda xd, bd, gd: K.in_forward(xd, bd, gd, 1e-5, channel_last=cl)
            bwd_r = lambda m, v, dm, dv: R.in_backward(x, dy, g, m, v, n, c, 1e-5, dm, dv)
            bwd_d = lambda xd, dyd, gd, m, v, **kw: K.in_backward(xd, dyd, gd, m, v, 1e-5, channel_last=cl, **kw)
    xd, dyd = to_dev(lay(x), dt), to_dev(lay(dy), dt)
    gd = to_dev(g) if g is not None else None
    bd = to_dev(b) if b is not None else None
    y_r, m_r, v_r = fwd_r()
    y, m, v = fwd_d(xd, bd, gd)
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(y), lay(np.asarray(y_r).reshape(x.shape)), dn, "y", "y")
    dm = f32(rng.standard_normal(nstat) * 0.3) if three else None
    dv = f32(rng.standard_normal(nstat) * 0.3) if three else None
    dx_r, dg_r, db_r = bwd_r(m_r, v_r, dm, dv)
    pre_dx = np.asarray(rounded(rng.standard_normal(x.shape), dt))
    pre_g = f32(rng.standard_normal(nparam))
    pre_b = f32(rng.standard_normal(nparam))
    dxd, dgd, dbd = to_dev(lay(pre_dx), dt), to_dev(pre_g), to_dev(pre_b)
    kw = dict(dx=dxd, dgamma=dgd, dbeta=dbd, accum=accum, need=need)
    if three:
        kw.update(dmean=to_dev(dm), dvar=to_dev(dv))
    bwd_d(xd, dyd, gd, m, v, **kw)
    torch.cuda.synchronize()
    exp_dx = np.asarray(dx_r).reshape(x.shape) + (pre_dx if accum[0] else 0) if need[0] else pre_dx
    exp_g = (dg_r + (pre_g if accum[1] else 0)) if need[1] else pre_g
    exp_b = (db_r + (pre_b if accum[2] else 0)) if need[2] else pre_b
    assert_close(to_np(dxd), lay(exp_dx), dn, "grad", "dx")
    assert_close(to_np(dgd), exp_g, dn, "pgrad", "dgamma")
    assert_close(to_np(dbd), exp_b, dn, "pgrad", "dbeta")


@pytest.mark.parametrize("seed", range(160))
def test_random_flags(seed):
    K.tune_reset()
    try:
        one_case(np.random.default_rng(11000 + seed))
    except AssertionError as e:
        raise AssertionError(f"{dict(LAST_CASE)}: {e}") from None
