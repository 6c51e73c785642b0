"""In-place calls (y == x, dx == dy, dx == x) on the shapes whose default plan
is a kernel family in which blocks exchange partial sums.  Such a block, when
a partner's word does not arrive in time, reads the partner's part of the
inputs again; in place the partner may already have overwritten it.  The
plans therefore turn in-place calls down and a kernel without an exchange
takes them.  Checked here: the out-of-place call of every shape does run the
exchanging kernel (so the shape is one the rule decides about), the in-place
call does not, and its results match the oracle, also with every poll
forbidden; an output that overlaps an input only in part is an error."""
import numpy as np
import pytest
import torch

from _util import assert_close, dtype_name, load_package, rounded, to_dev, to_np
from oracle import norm_ref as R

pytestmark = pytest.mark.gpu
K = load_package()
F32, F16 = torch.float32, torch.float16

EXCHANGING = {"bn_chan_split_fwd_kernel", "bn_chan_split_bwd_kernel", "bn_cl_grid_fwd_kernel",
              "bn_cl_grid_bwd_kernel", "cl_split_fwd_kernel", "cl_split_bwd_kernel",
              "gn_cl_tile_fwd_kernel", "gn_cl_tile_bwd_kernel"}


def f32(a):
    return np.asarray(a, np.float32).astype(np.float64)


@pytest.fixture(autouse=True)
def _default_knobs():
    K.tune_reset()
    yield
    K.tune_reset()
    K.check(K.lib().nblahip_profile_enable(0))


def traced(fn):
    K.check(K.lib().nblahip_profile_enable(64))
    out = fn()
    torch.cuda.synchronize()
    names = set(K.profile_kernels())
    K.check(K.lib().nblahip_profile_enable(0))
    return out, names


def to_cf(a):
    return np.ascontiguousarray(np.moveaxis(a, -1, 1))


def to_cl(a):
    return np.ascontiguousarray(np.moveaxis(a, 1, -1))


# BatchNormalization: (shape, axis, dtype, kernels of the out-of-place plan)
BN_CASES = [
    # fewer channels than CUs: a channel split over several blocks
    ((32, 64, 56, 56), 1, F16, "bn_chan_split"),
    ((37, 64, 32, 32), 1, F32, "bn_chan_split"),
    # channel-last, the whole tensor held on the chip
    ((200704, 64), 1, F16, "bn_cl_grid"),
    ((40000, 256), 1, F32, "bn_cl_grid"),
    # channel-last through the split kernels (all rows as one plane)
    ((32, 14, 14, 1024), 3, F16, "cl_split"),
]


@pytest.mark.parametrize("spin", [None, 0])
@pytest.mark.parametrize("shape,axis,dtype,family", BN_CASES)
def test_bn_in_place_takes_no_exchanging_kernel(shape, axis, dtype, family, spin):
    dn = dtype_name(dtype)
    rng = np.random.default_rng(5)
    c = shape[axis]
    x = rounded(rng.standard_normal(shape) * 1.5 + 0.5, dtype)
    dy = rounded(rng.standard_normal(shape), dtype)
    g, b = f32(rng.uniform(0.5, 1.5, c)), f32(rng.standard_normal(c) * 0.1)
    rm, rv = np.zeros(c), np.ones(c)
    y_r, m_r, v_r, rm_r, rv_r = R.bn_forward_batch(x, b, g, rm, rv, axis, 0.9, 1e-5)
    dx_r, dg_r, db_r = R.bn_backward_batch(x, dy, g, m_r, v_r, axis, 1e-5)
    gd, bd = to_dev(g), to_dev(b)
    if spin is not None:
        K.tune_set("XCHG_SPIN", spin)

    # out of place: the exchanging family runs
    xd, dyd = to_dev(x, dtype), to_dev(dy, dtype)
    (y, m, v), names = traced(lambda: K.bn_forward_batch(xd, bd, gd, to_dev(rm), to_dev(rv), axis, 0.9, 1e-5))
    assert family + "_fwd_kernel" in names, names
    (dx, dg, db), names = traced(lambda: K.bn_backward(xd, dyd, gd, m, v, axis, 1e-5))
    assert family + "_bwd_kernel" in names, names
    assert_close(to_np(y), y_r, dn, "y", "y")
    assert_close(to_np(dx), dx_r, dn, "grad", "dx")

    # y == x
    xi = xd.clone()
    rmd, rvd = to_dev(rm), to_dev(rv)
    (yi, mi, vi), names = traced(lambda: K.bn_forward_batch(xi, bd, gd, rmd, rvd, axis, 0.9, 1e-5, y=xi))
    assert not (names & EXCHANGING), names
    assert yi.data_ptr() == xi.data_ptr()
    assert_close(to_np(xi), y_r, dn, "y", "y in place")
    assert_close(to_np(mi), m_r, dn, "stat", "mean")
    assert_close(to_np(vi), v_r, dn, "stat", "var")
    assert_close(to_np(rvd), rv_r, dn, "stat", "running var")

    # dx == dy and dx == x
    for which in ("dy", "x"):
        xi, dyi = xd.clone(), dyd.clone()
        tgt = dyi if which == "dy" else xi
        (dxi, dgi, dbi), names = traced(lambda: K.bn_backward(xi, dyi, gd, m, v, axis, 1e-5, dx=tgt))
        assert not (names & EXCHANGING), names
        assert_close(to_np(tgt), dx_r, dn, "grad", "dx in place of " + which)
        assert_close(to_np(dgi), dg_r, dn, "pgrad", "dgamma")
        assert_close(to_np(dbi), db_r, dn, "pgrad", "dbeta")


# Channel-last Group / InstanceNormalization: (n, spatial, c, groups or None, dtype, family)
CL_CASES = [
    (3, (33, 33), 64, 8, F16, "cl_split"),
    (2, (70, 70), 64, 8, F32, "cl_split"),
    (2, (40, 40), 64, None, F16, "cl_split"),
    # groups that are no whole number of vectors: position tiles
    (2, (32, 32), 320, 32, F16, "gn_cl_tile"),
    (4, (16, 16), 640, 32, F32, "gn_cl_tile"),
]


@pytest.mark.parametrize("spin", [None, 0])
@pytest.mark.parametrize("n,sp,c,groups,dtype,family", CL_CASES)
def test_channel_last_in_place_takes_no_exchanging_kernel(n, sp, c, groups, dtype, family, spin):
    dn = dtype_name(dtype)
    rng = np.random.default_rng(6)
    shape = (n,) + sp + (c,)
    x = rounded(rng.standard_normal(shape) * 1.5 + rng.uniform(-2, 2, (n,) + (1,) * len(sp) + (c,)), dtype)
    dy = rounded(rng.standard_normal(shape), dtype)
    g, b = f32(rng.uniform(0.5, 1.5, c)), f32(rng.standard_normal(c) * 0.1)
    xt, dyt = to_cf(x), to_cf(dy)
    if groups is None:
        y_r, m_r, v_r = R.in_forward(xt, b, g, n, c, 1e-5)
        dx_r, dg_r, db_r = R.in_backward(xt, dyt, g, m_r, v_r, n, c, 1e-5)
        fwd = lambda xx, **kw: K.in_forward(xx, bd, gd, 1e-5, channel_last=True, **kw)
        bwd = lambda xx, dd, m, v, **kw: K.in_backward(xx, dd, gd, m, v, 1e-5, channel_last=True, **kw)
    else:
        y_r, m_r, v_r = R.gn_forward(xt, b, g, n, c, groups, 1e-5)
        dx_r, dg_r, db_r = R.gn_backward(xt, dyt, g, m_r, v_r, n, c, groups, 1e-5)
        fwd = lambda xx, **kw: K.gn_forward(xx, bd, gd, groups, 1e-5, channel_last=True, **kw)
        bwd = lambda xx, dd, m, v, **kw: K.gn_backward(xx, dd, gd, m, v, groups, 1e-5, channel_last=True, **kw)
    y_r = to_cl(np.asarray(y_r).reshape(xt.shape))
    dx_r = to_cl(np.asarray(dx_r).reshape(xt.shape))
    gd, bd = to_dev(g), to_dev(b)
    if spin is not None:
        K.tune_set("XCHG_SPIN", spin)

    xd, dyd = to_dev(x, dtype), to_dev(dy, dtype)
    (y, m, v), names = traced(lambda: fwd(xd))
    assert family + "_fwd_kernel" in names, names
    (dx, dg, db), names = traced(lambda: bwd(xd, dyd, m, v))
    assert family + "_bwd_kernel" in names, names
    assert_close(to_np(y), y_r, dn, "y", "y")
    assert_close(to_np(dx), dx_r, dn, "grad", "dx")

    xi = xd.clone()
    (yi, mi, vi), names = traced(lambda: fwd(xi, y=xi))
    assert not (names & EXCHANGING), names
    assert_close(to_np(xi), y_r, dn, "y", "y in place")
    assert_close(to_np(mi), np.asarray(m_r).ravel(), dn, "stat", "mean")
    assert_close(to_np(vi), np.asarray(v_r).ravel(), dn, "stat", "var")

    for which in ("dy", "x"):
        xi, dyi = xd.clone(), dyd.clone()
        tgt = dyi if which == "dy" else xi
        (dxi, dgi, dbi), names = traced(lambda: bwd(xi, dyi, m, v, dx=tgt))
        assert not (names & EXCHANGING), names
        assert_close(to_np(tgt), dx_r, dn, "grad", "dx in place of " + which)
        assert_close(to_np(dgi), dg_r, dn, "pgrad", "dgamma")
        assert_close(to_np(dbi), db_r, dn, "pgrad", "dbeta")


def test_partial_overlap_is_rejected():
    """An output that shares only part of its bytes with an input: NBLAHIP_EALIAS
    before anything is launched."""
    n, c, s = 4, 16, 64
    buf = torch.randn(2 * n * c * s + 64, device="cuda")
    x = buf[:n * c * s].view(n, c, s)
    y = buf[32:32 + n * c * s].view(n, c, s)
    g = torch.ones(c, device="cuda")
    b = torch.zeros(c, device="cuda")
    with pytest.raises(K.NblaHipError) as e:
        K.bn_forward_batch(x, b, g, torch.zeros(c, device="cuda"), torch.ones(c, device="cuda"), 1, 0.9,
                           1e-5, y=y)
    assert e.value.code == -4  # NBLAHIP_EALIAS
    m = torch.zeros(c, device="cuda")
    v = torch.ones(c, device="cuda")
    with pytest.raises(K.NblaHipError):
        K.bn_backward(x, x.clone(), g, m, v, 1, 1e-5, dx=y)
    xc = torch.randn(2, 16, 64, device="cuda")
    flat = torch.randn(2 * 16 * 64 + 64, device="cuda")
    yc = flat[16:16 + 2 * 16 * 64].view(2, 16, 64)
    xc2 = flat[:2 * 16 * 64].view(2, 16, 64)
    with pytest.raises(K.NblaHipError):
        K.gn_forward(xc2, torch.zeros(64, device="cuda"), torch.ones(64, device="cuda"), 8, 1e-5,
                     channel_last=True, y=yc)
