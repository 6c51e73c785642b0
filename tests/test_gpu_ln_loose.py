"""LayerNormalization over rows that are no whole number of 16-byte vectors,
or that start off a 16-byte boundary.  The backward of such rows of 64 to 256
vectors runs on a kernel that reads them with 16-byte accesses at element
alignment (ln_loose_bwd_kernel); the forward and longer rows stay with the row
kernels.  Parity against the oracle for every layout, flags, pointers at odd
offsets, and a guard band behind every output: the elements behind a row's
last whole vector are written one by one, so nothing may change behind the
tensor."""
import numpy as np
import pytest
import torch

from _util import assert_close, dtype_name, load_package, rounded, to_dev, to_np
from oracle import norm_ref as R

pytestmark = pytest.mark.gpu
K = load_package()
F32, F16 = torch.float32, torch.float16


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


def make(outer, Rr, dtype, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((outer, Rr)) * 1.5 + rng.uniform(-3, 3, (outer, 1))
    dy = rng.standard_normal((outer, Rr))
    g = f32(rng.standard_normal(Rr) * 0.1 + 1)
    b = f32(rng.standard_normal(Rr) * 0.1)
    return rounded(x, dtype), rounded(dy, dtype), g, b


def at_offset(a, dtype, off, guard=64):
    """Device tensor holding `a` at element offset `off` of a larger buffer whose
    other elements are a sentinel; returns (view, buffer)."""
    n = a.size
    buf = torch.full((off + n + guard,), 7.0, dtype=dtype, device="cuda")
    view = buf[off:off + n].view(a.shape)
    view.copy_(to_dev(a, dtype))
    return view, buf


def guard_intact(buf, off, n):
    return bool((buf[:off] == 7.0).all()) and bool((buf[off + n:] == 7.0).all())


# (rows, R, dtype): one wave per row with 1 / 2 / 4 vectors per lane, rows that
# end 1 .. VEC-1 elements behind their last whole vector, whole vectors at a
# shifted start, and longer rows (which the row kernels keep).
SHAPES = [
    (37, 513, F16), (300, 1023, F16), (64, 1028, F16), (33, 1004, F16), (19, 2047, F16),
    (21, 2049, F16), (9, 4100, F16), (5, 8191, F16), (3, 8201, F16), (2, 16383, F16),
    (40, 257, F32), (130, 1023, F32), (64, 1026, F32), (11, 2049, F32), (7, 4099, F32),
    (4, 8190, F32),
    # more rows than the persistent backward grid has row slots
    (5000, 1023, F16), (5000, 515, F32),
]


@pytest.mark.parametrize("off", [0, 1, 3])
@pytest.mark.parametrize("outer,Rr,dtype", SHAPES)
def test_forward_backward_at_element_alignment(outer, Rr, dtype, off):
    if outer >= 5000 and off:
        pytest.skip("offsets are covered by the smaller shapes")
    dn = dtype_name(dtype)
    x, dy, g, b = make(outer, Rr, dtype, 11)
    y_r, m_r, v_r = R.ln_forward(x, b, g, outer, 1e-5)
    dx_r, dg_r, db_r = R.ln_backward(x, dy, g, m_r, v_r, outer, 1e-5)
    xd, _ = at_offset(x, dtype, off)
    dyd, _ = at_offset(dy, dtype, off)
    gd, bd = to_dev(g), to_dev(b)
    yv, ybuf = at_offset(np.zeros_like(x), dtype, off)
    dxv, dxbuf = at_offset(np.zeros_like(x), dtype, off)
    L = K.lib()
    dt = K._dtype_code(xd)
    m = torch.empty(outer, device="cuda")
    v = torch.empty(outer, device="cuda")

    K.check(L.nblahip_ln_fwd(xd.data_ptr(), gd.data_ptr(), bd.data_ptr(), yv.data_ptr(), m.data_ptr(),
                             v.data_ptr(), outer, Rr, 1e-5, dt, None))
    torch.cuda.synchronize()
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(yv), y_r, dn, "y", "y")
    assert guard_intact(ybuf, off, x.size)

    dg = torch.empty(Rr, device="cuda")
    db = torch.empty(Rr, device="cuda")
    (_, _, _), names = traced(lambda: K.ln_backward(xd, dyd, gd, m, v, outer, 1e-5, dx=dxv, dgamma=dg, dbeta=db))
    vec = 8 if dtype == F16 else 4
    if 64 * vec <= Rr <= 256 * vec:
        assert names == {"ln_loose_bwd_kernel", "ln_param_reduce_kernel"}, names
    else:
        assert "ln_loose_bwd_kernel" not in names, names
    assert_close(to_np(dxv), dx_r, dn, "grad", "dx")
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")
    assert guard_intact(dxbuf, off, x.size)


@pytest.mark.parametrize("outer,Rr,dtype", [(33, 1023, F16), (20, 1022, F32), (6, 2044, F16)])
def test_flags(outer, Rr, dtype):
    """no_scale / no_bias, the three-output form, accumulation, propagate_down."""
    dn = dtype_name(dtype)
    x, dy, g, b = make(outer, Rr, dtype, 12)
    rng = np.random.default_rng(13)
    dm, dv = f32(rng.standard_normal(outer)), f32(rng.standard_normal(outer))
    xd, dyd = to_dev(x, dtype), to_dev(dy, dtype)
    y_r, m_r, v_r = R.ln_forward(x, None, None, outer, 1e-5)
    y, m, v = K.ln_forward(xd, None, None, outer, 1e-5)
    assert_close(to_np(y), y_r, dn, "y", "y no affine")
    dx_r, dg_r, db_r = R.ln_backward(x, dy, None, m_r, v_r, outer, 1e-5, dm, dv)
    (dx, dg, db), names = traced(lambda: K.ln_backward(xd, dyd, None, m, v, outer, 1e-5, dmean=to_dev(dm),
                                                        dvar=to_dev(dv)))
    assert "ln_loose_bwd_kernel" in names
    assert_close(to_np(dx), dx_r, dn, "grad", "dx three outputs")
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")

    dx_r, dg_r, db_r = R.ln_backward(x, dy, g, m_r, v_r, outer, 1e-5)
    pre_dx = rounded(rng.standard_normal((outer, Rr)), dtype)
    pre_g = f32(rng.standard_normal(Rr))
    pre_b = f32(rng.standard_normal(Rr))
    dxd, dgd, dbd = to_dev(pre_dx, dtype), to_dev(pre_g), to_dev(pre_b)
    K.ln_backward(xd, dyd, to_dev(g), m, v, outer, 1e-5, dx=dxd, dgamma=dgd, dbeta=dbd,
                  accum=(True, True, True))
    assert_close(to_np(dxd), dx_r + pre_dx, dn, "grad", "dx accum")
    assert_close(to_np(dgd), dg_r + pre_g, dn, "pgrad", "dgamma accum")
    assert_close(to_np(dbd), db_r + pre_b, dn, "pgrad", "dbeta accum")
    _, dg, db = K.ln_backward(xd, dyd, to_dev(g), m, v, outer, 1e-5, need=(False, True, True))
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma only")
    dx, _, _ = K.ln_backward(xd, dyd, to_dev(g), m, v, outer, 1e-5, need=(True, False, False))
    assert_close(to_np(dx), dx_r, dn, "grad", "dx only")


def test_in_place_and_determinism():
    """dx written over dy and over x (a wave has read the whole row before it
    writes any of it), and bit-equal repeats."""
    outer, Rr = 257, 1023
    x, dy, g, b = make(outer, Rr, F16, 14)
    y_r, m_r, v_r = R.ln_forward(x, b, g, outer, 1e-5)
    dx_r, dg_r, db_r = R.ln_backward(x, dy, g, m_r, v_r, outer, 1e-5)
    xd, dyd, gd = to_dev(x, F16), to_dev(dy, F16), to_dev(g)
    m, v = to_dev(f32(m_r)), to_dev(f32(v_r))
    dx1, dg1, db1 = K.ln_backward(xd, dyd, gd, m, v, outer, 1e-5)
    dx2, dg2, db2 = K.ln_backward(xd, dyd, gd, m, v, outer, 1e-5)
    assert torch.equal(dx1, dx2) and torch.equal(dg1, dg2) and torch.equal(db1, db2)
    for which in ("dy", "x"):
        xi, dyi = xd.clone(), dyd.clone()
        tgt = dyi if which == "dy" else xi
        (_, dgi, dbi), names = traced(lambda: K.ln_backward(xi, dyi, gd, m, v, outer, 1e-5, dx=tgt))
        assert "ln_loose_bwd_kernel" in names
        assert torch.equal(tgt, dx1), which
        assert torch.equal(dgi, dg1) and torch.equal(dbi, db1)
    assert_close(to_np(dx1), dx_r, "f16", "grad", "dx")


def test_switched_off_takes_the_scalar_rows():
    outer, Rr = 64, 1023
    x, dy, g, b = make(outer, Rr, F16, 15)
    xd, dyd, gd = to_dev(x, F16), to_dev(dy, F16), to_dev(g)
    y, m, v = K.ln_forward(xd, to_dev(b), gd, outer, 1e-5)
    K.tune_set("LN_LOOSE", 0)
    (dx0, dg0, db0), names = traced(lambda: K.ln_backward(xd, dyd, gd, m, v, outer, 1e-5))
    assert names == {"row_bwd_kernel_ln", "ln_param_reduce_kernel"}, names
    K.tune_reset()
    dx1, dg1, db1 = K.ln_backward(xd, dyd, gd, m, v, outer, 1e-5)
    assert_close(to_np(dx1), to_np(dx0).astype(np.float64), "f16", "grad", "dx against the scalar rows")
    assert_close(to_np(dg1), to_np(dg0).astype(np.float64), "f16", "pgrad", "dgamma against the scalar rows")
