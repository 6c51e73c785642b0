"""Tensor layouts the normalization kernels do not read in place: Group and
InstanceNormalization with the channel axis in the middle or before a batch
axis, LayerNormalization with batch axes that are not the leading ones.  The
Function classes bring them to the kernels' layout with a device permutation
and back (the reference uses the core's ChannelFirstAdaptor and the core's own
function for these, group_normalization.cu:40-55, instance_normalization.cu:
40-51, layer_normalization.cu:43-51).  Every case is compared with the oracle
on the transposed tensor, statistics and parameter gradients in the caller's
axis order."""
import numpy as np
import pytest

from _util import assert_close, load_package
from oracle import norm_ref as R

load_package()
from nnabla_ext_cuda_amd import binding as B  # noqa: E402

pytestmark = pytest.mark.gpu
CONFIGS = ["float", "half"]


def dn(tc):
    return "f16" if tc == "half" else "f32"


def rnd(a, tc):
    a = np.asarray(a, np.float32)
    return a.astype(np.float16).astype(np.float64) if tc == "half" else a.astype(np.float64)


def var(a, half=False):
    v = B.Variable(np.shape(a))
    v.set_data(a, half=half)
    return v


@pytest.fixture(scope="module", autouse=True)
def _init():
    B.init()


def _front_perm(ndim, front):
    return list(front) + [i for i in range(ndim) if i not in front]


# (shape, batch_axis, channel_axis, groups)
GN_CASES = [
    ((4, 6, 8, 5), [0], 2, 4),       # channel axis in the middle
    ((3, 5, 7, 12, 4), [0], 3, 3),
    ((2, 3, 5, 16, 6), [0, 1], 3, 8),  # two batch axes, channel behind a spatial axis
    ((8, 4, 9), [1], 0, 2),          # channel axis before the batch axis
    ((5, 6, 2, 7), [2], 1, 3),       # batch axis in the middle
    ((2, 70, 16, 33), [0], 2, 4),    # several tiles per axis in the permutation
]


@pytest.mark.parametrize("tc", CONFIGS)
@pytest.mark.parametrize("shape,batch_axis,c_axis,groups", GN_CASES)
def test_group_normalization_any_layout(tc, shape, batch_axis, c_axis, groups):
    rng = np.random.default_rng(31)
    half = tc == "half"
    nd = len(shape)
    c = shape[c_axis]
    n = int(np.prod([shape[b] for b in batch_axis]))
    pshape = tuple(c if i == c_axis else 1 for i in range(nd))
    x = rnd(rng.standard_normal(shape) * 1.5 + 0.3, tc)
    dy = rnd(rng.standard_normal(shape), tc)
    g = rng.uniform(0.5, 1.5, pshape).astype(np.float32)
    b = (rng.standard_normal(pshape) * 0.1).astype(np.float32)
    f = B.GroupNormalization(B.context(type_config=tc), num_groups=groups, channel_axis=c_axis,
                             batch_axis=list(batch_axis))
    vx, vb, vg = var(x, half), var(b), var(g)
    vy, om, ov = B.Variable(shape), B.Variable(()), B.Variable(())
    f.setup([vx, vb, vg], [vy, om, ov])
    f.forward([vx, vb, vg], [vy, om, ov])
    perm = _front_perm(nd, sorted(batch_axis) + [c_axis])
    inv = np.argsort(perm)
    xt, dyt = np.transpose(x, perm), np.transpose(dy, perm)
    y_r, m_r, v_r = R.gn_forward(xt, b, g, n, c, groups, 1e-5)
    back = lambda a: np.transpose(np.asarray(a).reshape(xt.shape), inv)
    # statistics [batch..., groups] -> the caller's axis order
    kept = sorted(list(batch_axis) + [c_axis])
    kshape = [shape[b] for b in sorted(batch_axis)] + [groups]
    kperm = [(sorted(batch_axis) + [c_axis]).index(k) for k in kept]
    to_caller = lambda a: np.transpose(np.asarray(a).reshape(kshape), kperm)
    to_kernel = lambda a: np.transpose(np.asarray(a).reshape([kshape[i] for i in kperm]),
                                       np.argsort(kperm)).reshape(-1)
    assert_close(vy.d, back(y_r), dn(tc), "y", "y")
    assert_close(om.d, to_caller(m_r), dn(tc), "stat", "mean output")
    assert_close(ov.d, to_caller(v_r), dn(tc), "stat", "var output")
    dm = rng.standard_normal(om.current_shape).astype(np.float32)
    dv = rng.standard_normal(ov.current_shape).astype(np.float32)
    pre = rnd(rng.standard_normal(shape), tc)
    vy.set_grad(dy, half)
    om.set_grad(dm)
    ov.set_grad(dv)
    vx.set_grad(pre, half)
    f.backward([vx, vb, vg], [vy, om, ov], propagate_down=[1, 1, 1], accum=[1, 0, 0])
    dx_r, dg_r, db_r = R.gn_backward(xt, dyt, g, m_r, v_r, n, c, groups, 1e-5, to_kernel(dm),
                                     to_kernel(dv))
    assert_close(vx.g, back(dx_r) + pre, dn(tc), "grad", "dx accumulated")
    assert_close(vg.g, dg_r, dn(tc), "pgrad", "dgamma")
    assert_close(vb.g, db_r, dn(tc), "pgrad", "dbeta")
    # one output, dx overwritten
    vy1 = B.Variable(shape)
    f.setup([vx, vb, vg], [vy1])
    f.forward([vx, vb, vg], [vy1])
    assert_close(vy1.d, back(y_r), dn(tc), "y", "y, one output")
    vy1.set_grad(dy, half)
    f.backward([vx, vb, vg], [vy1], propagate_down=[1, 0, 0], accum=[0, 0, 0])
    dx1, _, _ = R.gn_backward(xt, dyt, g, m_r, v_r, n, c, groups, 1e-5)
    assert_close(vx.g, back(dx1), dn(tc), "grad", "dx")


IN_CASES = [
    ((4, 6, 8, 5), [0], 2),
    ((2, 3, 5, 16, 6), [0, 1], 3),
    ((8, 4, 9), [1], 0),
    ((5, 6, 2, 7), [2], 1),
    ((2, 70, 16, 33), [0], 2),
]


@pytest.mark.parametrize("tc", CONFIGS)
@pytest.mark.parametrize("per_sample", [False, True])
@pytest.mark.parametrize("shape,batch_axis,c_axis", IN_CASES)
def test_instance_normalization_any_layout(tc, per_sample, shape, batch_axis, c_axis):
    rng = np.random.default_rng(32)
    half = tc == "half"
    nd = len(shape)
    c = shape[c_axis]
    n = int(np.prod([shape[b] for b in batch_axis]))
    pshape = tuple(shape[i] if (i == c_axis or (per_sample and i in batch_axis)) else 1
                   for i in range(nd))
    x = rnd(rng.standard_normal(shape) * 1.5 + 0.3, tc)
    dy = rnd(rng.standard_normal(shape), tc)
    g = rng.uniform(0.5, 1.5, pshape).astype(np.float32)
    b = (rng.standard_normal(pshape) * 0.1).astype(np.float32)
    f = B.InstanceNormalization(B.context(type_config=tc), channel_axis=c_axis,
                                batch_axis=list(batch_axis))
    vx, vb, vg = var(x, half), var(b), var(g)
    vy, om, ov = B.Variable(shape), B.Variable(()), B.Variable(())
    f.setup([vx, vb, vg], [vy, om, ov])
    f.forward([vx, vb, vg], [vy, om, ov])
    front = sorted(batch_axis) + [c_axis]
    perm = _front_perm(nd, front)
    inv = np.argsort(perm)
    xt, dyt = np.transpose(x, perm), np.transpose(dy, perm)
    back = lambda a: np.transpose(np.asarray(a).reshape(xt.shape), inv)
    # [batch..., channel] <-> the caller's axis order of those axes
    kept = sorted(front)
    kshape = [shape[k] for k in front]
    kperm = [front.index(k) for k in kept]
    to_caller = lambda a: np.transpose(np.asarray(a).reshape(kshape), kperm)
    to_kernel = lambda a: np.transpose(np.asarray(a).reshape([kshape[i] for i in kperm]),
                                       np.argsort(kperm)).reshape(-1)
    gk = to_kernel(g) if per_sample else g.reshape(-1)
    bk = to_kernel(b) if per_sample else b.reshape(-1)
    g_full = gk if per_sample else np.tile(gk, n)
    b_full = bk if per_sample else np.tile(bk, n)
    y_r, m_r, v_r = R.in_forward(xt, b_full, g_full, n, c, 1e-5)
    assert_close(vy.d, back(y_r), dn(tc), "y", "y")
    assert_close(om.d, to_caller(m_r), dn(tc), "stat", "mean output")
    assert_close(ov.d, to_caller(v_r), dn(tc), "stat", "var output")
    dm = rng.standard_normal(om.current_shape).astype(np.float32)
    dv = rng.standard_normal(ov.current_shape).astype(np.float32)
    pre_g = rng.standard_normal(pshape).astype(np.float32)
    vy.set_grad(dy, half)
    om.set_grad(dm)
    ov.set_grad(dv)
    vg.set_grad(pre_g)
    f.backward([vx, vb, vg], [vy, om, ov], propagate_down=[1, 1, 1], accum=[0, 0, 1])
    dx_r, dg_r, db_r = R.in_backward(xt, dyt, gk, m_r, v_r, n, c, 1e-5, to_kernel(dm),
                                     to_kernel(dv), bc_gamma=not per_sample,
                                     bc_beta=not per_sample)
    if per_sample:
        dg_r, db_r = to_caller(dg_r), to_caller(db_r)
    assert_close(vx.g, back(dx_r), dn(tc), "grad", "dx")
    assert_close(vg.g, np.asarray(dg_r).reshape(-1) + pre_g.reshape(-1), dn(tc), "pgrad",
                 "dgamma accumulated")
    assert_close(vb.g, db_r, dn(tc), "pgrad", "dbeta")


LN_CASES = [
    ((4, 6, 8), [1]),
    ((4, 6, 8), [2]),
    ((4, 6, 8, 5), [0, 2]),
    ((4, 6, 8, 5), [1, 3]),
    ((3, 5, 7, 2, 4), [4, 1]),
    ((2, 130, 3, 70), [1]),
    ((6, 1, 8), [1]),                 # only an axis of extent 1 moves: read in place
]


@pytest.mark.parametrize("tc", CONFIGS)
@pytest.mark.parametrize("shape,batch_axis", LN_CASES)
def test_layer_normalization_any_batch_axes(tc, shape, batch_axis):
    rng = np.random.default_rng(33)
    half = tc == "half"
    nd = len(shape)
    ba = sorted(batch_axis)
    outer = int(np.prod([shape[b] for b in ba]))
    pshape = tuple(1 if i in ba else s for i, s in enumerate(shape))
    x = rnd(rng.standard_normal(shape) + rng.uniform(-3, 3, [s if i in ba else 1 for i, s in
                                                              enumerate(shape)]), tc)
    dy = rnd(rng.standard_normal(shape), tc)
    g = (rng.standard_normal(pshape) * 0.1 + 1).astype(np.float32)
    b = (rng.standard_normal(pshape) * 0.1).astype(np.float32)
    f = B.LayerNormalization(B.context(type_config=tc), batch_axis=list(batch_axis), eps=1e-5)
    vx, vb, vg = var(x, half), var(b), var(g)
    vy, om, ov = B.Variable(shape), B.Variable(()), B.Variable(())
    f.setup([vx, vb, vg], [vy, om, ov])
    assert tuple(om.current_shape) == tuple(s if i in ba else 1 for i, s in enumerate(shape))
    f.forward([vx, vb, vg], [vy, om, ov])
    perm = _front_perm(nd, ba)
    inv = np.argsort(perm)
    xt, dyt = np.transpose(x, perm), np.transpose(dy, perm)
    back = lambda a: np.transpose(np.asarray(a).reshape(xt.shape), inv)
    y_r, m_r, v_r = R.ln_forward(xt, b, g, outer, 1e-5)
    assert_close(vy.d, back(y_r), dn(tc), "y", "y")
    assert_close(om.d, m_r, dn(tc), "stat", "mean output")
    assert_close(ov.d, v_r, dn(tc), "stat", "var output")
    dm = rng.standard_normal(om.current_shape).astype(np.float32)
    dv = rng.standard_normal(ov.current_shape).astype(np.float32)
    pre = rnd(rng.standard_normal(shape), tc)
    vy.set_grad(dy, half)
    om.set_grad(dm)
    ov.set_grad(dv)
    vx.set_grad(pre, half)
    f.backward([vx, vb, vg], [vy, om, ov], propagate_down=[1, 1, 1], accum=[1, 0, 0])
    dx_r, dg_r, db_r = R.ln_backward(xt, dyt, g, m_r, v_r, outer, 1e-5, dm, dv)
    assert_close(vx.g, back(dx_r) + pre, dn(tc), "grad", "dx accumulated")
    assert_close(vg.g, dg_r, dn(tc), "pgrad", "dgamma")
    assert_close(vb.g, db_r, dn(tc), "pgrad", "dbeta")
    f.backward([vx, vb, vg], [vy, om, ov], propagate_down=[1, 0, 0], accum=[0, 0, 0])
    assert_close(vx.g, back(dx_r), dn(tc), "grad", "dx")
