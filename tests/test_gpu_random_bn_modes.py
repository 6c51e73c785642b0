"""Randomly drawn BatchNormalization calls beyond the plain training step
(fixed seeds): FusedBatchNormalization with and without the residual input,
batch statistics or the running ones (inference-mode forward and backward),
both layouts and dtypes, tensors of 20 KB - 24 MB, the three-output gradients,
each of dx / dz / dgamma / dbeta wanted or not and accumulated or overwritten,
the running statistics after the call - against the oracle.  The gate of the
fused backward takes the device's own y, as the function does."""
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


def logi(rng, lo, hi):
    return int(np.exp(rng.uniform(np.log(lo), np.log(hi))))


def one_case(rng):
    dt = F16 if rng.integers(0, 2) else F32
    dn = dtype_name(dt)
    esz = 2 if dt == F16 else 4
    target = logi(rng, 2e4, 24e6) // esz
    cl = bool(rng.integers(0, 2))
    batch_stat = rng.random() < 0.7
    fused = rng.random() < 0.7
    use_z = fused and rng.random() < 0.7
    three = batch_stat and rng.random() < 0.4
    c = int(rng.choice([3, 8, 16, 24, 32, 40, 64, 72, 96, 100, 128, 200, 256, 320, 512, 1024, 2048]))
    h = int(rng.choice([1, 4, 7, 8, 14, 16, 17, 28, 32, 35, 56, 63, 64, 96]))
    w = h if rng.integers(0, 4) else int(rng.integers(1, 80))
    n = max(2, min(256, target // (h * w * c)))
    if n * h * w < 6:
        n = 6
    shape = (n, c, h, w)
    nn = 4 if fused else 3
    accum = tuple(bool(rng.integers(0, 2)) for _ in range(nn))
    need = tuple(bool(rng.random() > 0.25) for _ in range(nn))
    if not any(need):
        need = (True,) * nn
    desc = dict(dt=dn, cl=cl, batch_stat=batch_stat, fused=fused, z=use_z, three=three, shape=shape, accum=accum, need=need)
    LAST_CASE.clear()
    LAST_CASE.update(desc)
    axis = 3 if cl else 1
    lay = (lambda a: np.ascontiguousarray(np.moveaxis(a, 1, -1))) if cl else (lambda a: a)
    x = rounded(rng.standard_normal(shape) * 1.5 + rng.uniform(-2, 2, (1, c, 1, 1)), dt)
    dy = rounded(rng.standard_normal(shape), dt)
    z = rounded(rng.standard_normal(shape), dt) if use_z else None
    g = f32(rng.uniform(0.5, 1.5, c))
    b = f32(rng.standard_normal(c) * 0.3)
    rm, rv = f32(rng.standard_normal(c) * 0.5), f32(rng.uniform(0.5, 2.0, c))
    xd, dyd = to_dev(lay(x), dt), to_dev(lay(dy), dt)
    zd = to_dev(lay(z), dt) if use_z else None
    gd, bd, rmd, rvd = to_dev(g), to_dev(b), to_dev(rm), to_dev(rv)
    if fused:
        y_r, m_r, v_r, rm_r, rv_r = R.fused_bn_forward(x, z, b, g, rm, rv, 1, 0.9, 1e-5, batch_stat)
        if batch_stat:
            y, m, v = K.fused_bn_forward_batch(xd, zd, bd, gd, rmd, rvd, axis, 0.9, 1e-5)
        else:
            y = K.fused_bn_forward_global(xd, zd, bd, gd, rmd, rvd, axis, 1e-5)
    else:
        if batch_stat:
            y_r, m_r, v_r, rm_r, rv_r = R.bn_forward_batch(x, b, g, rm, rv, 1, 0.9, 1e-5)
            y, m, v = K.bn_forward_batch(xd, bd, gd, rmd, rvd, axis, 0.9, 1e-5)
        else:
            y_r = R.bn_forward_global(x, b, g, rm, rv, 1, 1e-5)
            y = K.bn_forward_global(xd, bd, gd, rmd, rvd, axis, 1e-5)
    assert_close(to_np(y), lay(np.asarray(y_r).reshape(shape)), dn, "y", "y")
    if batch_stat:
        assert_close(to_np(m), m_r, dn, "stat", "mean")
        assert_close(to_np(v), v_r, dn, "stat", "var")
        assert_close(to_np(rmd), rm_r, dn, "stat", "running mean")
        assert_close(to_np(rvd), rv_r, dn, "stat", "running var")
        mm, vv, mdev, vdev = m_r, v_r, m, v
    else:
        mm, vv, mdev, vdev = rm, rv, rmd, rvd
        assert_close(to_np(rmd), rm, dn, "stat", "running mean untouched")
    dm = f32(rng.standard_normal(c) * 0.3) if three else None
    dv = f32(rng.standard_normal(c) * 0.3) if three else None
    pre_dx = np.asarray(rounded(rng.standard_normal(shape), dt))
    pre_dz = np.asarray(rounded(rng.standard_normal(shape), dt))
    pre_g = f32(rng.standard_normal(c))
    pre_b = f32(rng.standard_normal(c))
    dxd, dzd, dgd, dbd = to_dev(lay(pre_dx), dt), to_dev(lay(pre_dz), dt), to_dev(pre_g), to_dev(pre_b)
    kw = {}
    if three:
        kw.update(dmean=to_dev(dm), dvar=to_dev(dv))
    if fused:
        y_host = np.moveaxis(to_np(y), -1, 1) if cl else to_np(y)
        dx_r, dz_r, dg_r, db_r = R.fused_bn_backward(x, y_host, dy, g, mm, vv, 1, 1e-5, batch_stat, dm, dv)
        K.fused_bn_backward(xd, y, dyd, gd, mdev, vdev, axis, 1e-5, batch_stat=batch_stat, dx=dxd, dz=dzd,
                            dgamma=dgd, dbeta=dbd, accum=accum, need=need, **kw)
        nd = dict(dx=(need[0], accum[0]), dz=(need[1], accum[1]), dg=(need[2], accum[2]), db=(need[3], accum[3]))
    else:
        if batch_stat:
            dx_r, dg_r, db_r = R.bn_backward_batch(x, dy, g, mm, vv, 1, 1e-5, dm, dv)
        else:
            dx_r, dg_r, db_r = R.bn_backward_global(x, dy, g, mm, vv, 1, 1e-5)
        K.bn_backward(xd, dyd, gd, mdev, vdev, axis, 1e-5, batch_stat=batch_stat, dx=dxd, dgamma=dgd, dbeta=dbd,
                      accum=accum, need=need, **kw)
        dz_r = None
        nd = dict(dx=(need[0], accum[0]), dz=(False, False), dg=(need[1], accum[1]), db=(need[2], accum[2]))
    torch.cuda.synchronize()

    def expect(ref, pre, key):
        nd_, ac_ = nd[key]
        if not nd_:
            return pre
        return np.asarray(ref).reshape(pre.shape) + (pre if ac_ else 0)

    assert_close(to_np(dxd), lay(expect(dx_r, pre_dx, "dx")), dn, "grad", "dx")
    assert_close(to_np(dzd), lay(expect(dz_r, pre_dz, "dz")), dn, "grad", "dz")
    assert_close(to_np(dgd), expect(dg_r, pre_g, "dg"), dn, "pgrad", "dgamma")
    assert_close(to_np(dbd), expect(db_r, pre_b, "db"), dn, "pgrad", "dbeta")


@pytest.mark.parametrize("seed", range(120))
def test_random_fused_and_inference_bn(seed):
    K.tune_reset()
    try:
        one_case(np.random.default_rng(13000 + seed))
    except AssertionError as e:
        raise AssertionError(f"{dict(LAST_CASE)}: {e}") from None
