"""The nbla::Function classes of the "hip" backend, driven the way NNabla's
function tests drive a backend: create by name and context, setup, forward,
backward with propagate_down/accum flags, compared with the oracle."""
import numpy as np
import pytest
import torch

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


@pytest.mark.parametrize("tc", CONFIGS)
@pytest.mark.parametrize("shape,axis", [((4, 8, 6, 6), 1), ((6, 5, 4, 8), 3), ((16, 24), 1)])
def test_batch_normalization_training(tc, shape, axis):
    rng = np.random.default_rng(1)
    half = tc == "half"
    c = shape[axis]
    pshape = tuple(c if i == axis else 1 for i in range(len(shape)))
    x = rnd(rng.standard_normal(shape) * 2 + 1, tc)
    dy = rnd(rng.standard_normal(shape), tc)
    g = rng.uniform(0.5, 1.5, pshape).astype(np.float32)
    b = (rng.standard_normal(pshape) * 0.1).astype(np.float32)
    rm = np.zeros(pshape, np.float32)
    rv = np.ones(pshape, np.float32)
    f = B.BatchNormalization(B.context(type_config=tc), axes=[axis], decay_rate=0.9, eps=1e-5, batch_stat=True)
    assert f.name == "BatchNormalizationHip"
    vx, vb, vg, vm, vv = var(x, half), var(b), var(g), var(rm), var(rv)
    vy = B.Variable(shape)
    ins = [vx, vb, vg, vm, vv]
    f.setup(ins, [vy])
    f.forward(ins, [vy])
    y_r, m_r, v_r, rm_r, rv_r = R.bn_forward_batch(x, b, g, rm, rv, axis, 0.9, 1e-5)
    assert_close(vy.d, y_r, dn(tc), "y", "y")
    assert_close(vm.d, rm_r, dn(tc), "stat", "running mean (updated in place)")
    assert_close(vv.d, rv_r, dn(tc), "stat", "running var (updated in place)")

    # recompute must not touch the running statistics
    f.recompute(ins, [vy])
    assert_close(vm.d, rm_r, dn(tc), "stat", "running mean after recompute")
    assert_close(vy.d, y_r, dn(tc), "y", "y after recompute")

    vy.set_grad(dy, half)
    f.backward(ins, [vy], propagate_down=[1, 1, 1, 0, 0], accum=[0, 0, 0, 0, 0])
    dx_r, dg_r, db_r = R.bn_backward_batch(x, dy, g, m_r, v_r, axis, 1e-5)
    assert_close(vx.g, dx_r, dn(tc), "grad", "dx")
    assert_close(vg.g, dg_r, dn(tc), "pgrad", "dgamma")
    assert_close(vb.g, db_r, dn(tc), "pgrad", "dbeta")

    # accumulation: run backward again onto the existing gradients
    f.backward(ins, [vy], propagate_down=[1, 1, 1, 0, 0], accum=[1, 1, 1, 0, 0])
    assert_close(vx.g, 2 * dx_r, dn(tc), "grad", "dx accum")
    assert_close(vg.g, 2 * dg_r, dn(tc), "pgrad", "dgamma accum")
    # propagate_down subset: only beta; the others keep their values
    before = vx.g.copy()
    f.backward(ins, [vy], propagate_down=[0, 1, 0, 0, 0], accum=[0, 0, 0, 0, 0])
    assert_close(vb.g, db_r, dn(tc), "pgrad", "dbeta only")
    np.testing.assert_array_equal(vx.g, before)


@pytest.mark.parametrize("tc", CONFIGS)
def test_batch_normalization_three_outputs_and_flags(tc):
    rng = np.random.default_rng(2)
    half = tc == "half"
    shape, axis, c = (4, 6, 5, 5), 1, 6
    pshape = (1, c, 1, 1)
    x = rnd(rng.standard_normal(shape), tc)
    dy = rnd(rng.standard_normal(shape), tc)
    dm = rng.standard_normal(pshape).astype(np.float32)
    dv = rng.standard_normal(pshape).astype(np.float32)
    rm, rv = np.zeros(pshape, np.float32), np.ones(pshape, np.float32)
    f = B.BatchNormalization(B.context(type_config=tc), axes=[axis], batch_stat=True, no_scale=True, no_bias=True)
    vx, vm, vv = var(x, half), var(rm), var(rv)
    vy, om, ov = B.Variable(shape), B.Variable(()), B.Variable(())
    f.setup([vx, vm, vv], [vy, om, ov])
    assert om.current_shape == pshape and ov.current_shape == pshape
    f.forward([vx, vm, vv], [vy, om, ov])
    y_r, m_r, v_r, _, _ = R.bn_forward_batch(x, None, None, None, None, axis, 0.9, 1e-5)
    assert_close(vy.d, y_r, dn(tc), "y", "y")
    assert_close(om.d, m_r, dn(tc), "stat", "mean output")
    assert_close(ov.d, v_r, dn(tc), "stat", "var output")
    vy.set_grad(dy, half)
    om.set_grad(dm)
    ov.set_grad(dv)
    f.backward([vx, vm, vv], [vy, om, ov], propagate_down=[1, 0, 0], accum=[0, 0, 0])
    dx_r, _, _ = R.bn_backward_batch(x, dy, None, m_r, v_r, axis, 1e-5, dm, dv)
    assert_close(vx.g, dx_r, dn(tc), "grad", "dx with dmean/dvar")


@pytest.mark.parametrize("tc", CONFIGS)
def test_batch_normalization_inference(tc):
    rng = np.random.default_rng(3)
    half = tc == "half"
    shape, c = (8, 16, 7, 7), 16
    pshape = (1, c, 1, 1)
    x = rnd(rng.standard_normal(shape), tc)
    dy = rnd(rng.standard_normal(shape), tc)
    g = rng.uniform(0.5, 1.5, pshape).astype(np.float32)
    b = (rng.standard_normal(pshape) * 0.1).astype(np.float32)
    rm = (rng.standard_normal(pshape) * 0.1).astype(np.float32)
    rv = rng.uniform(0.5, 2, pshape).astype(np.float32)
    f = B.BatchNormalization(B.context(type_config=tc), axes=[1], batch_stat=False)
    vx, vb, vg, vm, vv = var(x, half), var(b), var(g), var(rm), var(rv)
    vy = B.Variable(shape)
    ins = [vx, vb, vg, vm, vv]
    f.setup(ins, [vy])
    f.forward(ins, [vy])
    assert_close(vy.d, R.bn_forward_global(x, b, g, rm, rv, 1, 1e-5), dn(tc), "y", "y")
    np.testing.assert_array_equal(vm.d, rm)          # running stats are read-only here
    vy.set_grad(dy, half)
    f.backward(ins, [vy], propagate_down=[1, 1, 1, 0, 0], accum=[0] * 5)
    dx_r, dg_r, db_r = R.bn_backward_global(x, dy, g, rm, rv, 1, 1e-5)
    assert_close(vx.g, dx_r, dn(tc), "grad", "dx")
    assert_close(vg.g, dg_r, dn(tc), "pgrad", "dgamma")
    assert_close(vb.g, db_r, dn(tc), "pgrad", "dbeta")


@pytest.mark.parametrize("tc", CONFIGS)
@pytest.mark.parametrize("shape,axis", [((4, 8, 7, 7), 1), ((4, 7, 7, 16), 3)])
@pytest.mark.parametrize("with_z", [True, False])
def test_fused_batch_normalization(tc, shape, axis, with_z):
    """y = relu(bn(x) + z): forward with running-stat update, recompute,
    backward to x, beta, gamma and z, accumulation on z."""
    rng = np.random.default_rng(21)
    half = tc == "half"
    c = shape[axis]
    pshape = tuple(c if i == axis else 1 for i in range(len(shape)))
    x = rnd(rng.standard_normal(shape) * 2 + 1, tc)
    z = rnd(rng.standard_normal(shape), tc)
    dy = rnd(rng.standard_normal(shape), tc)
    g = rng.uniform(0.5, 1.5, pshape).astype(np.float32)
    b = (rng.standard_normal(pshape) * 0.3).astype(np.float32)
    rm, rv = np.zeros(pshape, np.float32), np.ones(pshape, np.float32)
    f = B.FusedBatchNormalization(B.context(type_config=tc), axes=[axis], decay_rate=0.9, eps=1e-5,
                                  batch_stat=True, nonlinearity="relu")
    assert f.name == "FusedBatchNormalizationHip"
    vx, vb, vg, vm, vv, vz = var(x, half), var(b), var(g), var(rm), var(rv), var(z, half)
    ins = [vx, vb, vg, vm, vv] + ([vz] if with_z else [])
    vy = B.Variable(shape)
    f.setup(ins, [vy])
    f.forward(ins, [vy])
    y_r, m_r, v_r, rm_r, rv_r = R.fused_bn_forward(x, z if with_z else None, b, g, rm, rv, axis,
                                                   0.9, 1e-5, True)
    assert_close(vy.d, y_r, dn(tc), "y", "y")
    assert_close(vm.d, rm_r, dn(tc), "stat", "running mean")
    assert_close(vv.d, rv_r, dn(tc), "stat", "running var")
    f.recompute(ins, [vy])
    assert_close(vm.d, rm_r, dn(tc), "stat", "running mean after recompute")
    y_gpu = vy.d.astype(np.float64)
    vy.set_grad(dy, half)
    n_in = len(ins)
    pd = [1, 1, 1, 0, 0] + ([1] if with_z else [])
    f.backward(ins, [vy], propagate_down=pd, accum=[0] * n_in)
    dx_r, dz_r, dg_r, db_r = R.fused_bn_backward(x, y_gpu, dy, g, m_r, v_r, axis, 1e-5, True)
    assert_close(vx.g, dx_r, dn(tc), "grad", "dx")
    assert_close(vg.g, dg_r, dn(tc), "pgrad", "dgamma")
    assert_close(vb.g, db_r, dn(tc), "pgrad", "dbeta")
    if with_z:
        np.testing.assert_array_equal(vz.g.astype(np.float64), dz_r)
        f.backward(ins, [vy], propagate_down=[0, 0, 0, 0, 0, 1], accum=[0, 0, 0, 0, 0, 1])
        assert_close(vz.g, 2 * dz_r, dn(tc), "grad", "dz accum")


@pytest.mark.parametrize("tc", CONFIGS)
def test_fused_batch_normalization_inference_and_errors(tc):
    rng = np.random.default_rng(22)
    half = tc == "half"
    shape, axis, c = (4, 6, 5, 5), 1, 6
    pshape = (1, c, 1, 1)
    x = rnd(rng.standard_normal(shape), tc)
    z = rnd(rng.standard_normal(shape), tc)
    g = rng.uniform(0.5, 1.5, pshape).astype(np.float32)
    b = (rng.standard_normal(pshape) * 0.3).astype(np.float32)
    rm = (rng.standard_normal(pshape) * 0.1).astype(np.float32)
    rv = rng.uniform(0.5, 2, pshape).astype(np.float32)
    f = B.FusedBatchNormalization(B.context(type_config=tc), axes=[axis], batch_stat=False)
    ins = [var(x, half), var(b), var(g), var(rm), var(rv), var(z, half)]
    vy = B.Variable(shape)
    f.setup(ins, [vy])
    f.forward(ins, [vy])
    y_r, _, _, _, _ = R.fused_bn_forward(x, z, b, g, rm, rv, axis, 0.9, 1e-5, False)
    assert_close(vy.d, y_r, dn(tc), "y", "y")
    np.testing.assert_array_equal(ins[3].d, rm)
    bad = B.FusedBatchNormalization(B.context(type_config=tc), axes=[axis], nonlinearity="tanh")
    with pytest.raises(B.NblaError, match="relu"):
        bad.setup(ins, [vy])
    few = B.FusedBatchNormalization(B.context(type_config=tc), axes=[axis])
    with pytest.raises(B.NblaError, match="at least 5 inputs"):
        few.setup(ins[:3], [vy])


@pytest.mark.parametrize("tc", CONFIGS)
@pytest.mark.parametrize("shape,batch_axis", [((4, 6, 64), (0, 1)), ((8, 1000), (0,)), ((3, 5, 7, 16), (0,))])
def test_layer_normalization(tc, shape, batch_axis):
    rng = np.random.default_rng(4)
    half = tc == "half"
    outer = int(np.prod([shape[a] for a in batch_axis]))
    pshape = tuple(1 if i in batch_axis else s for i, s in enumerate(shape))
    x = rnd(rng.standard_normal(shape) + 2, tc)
    dy = rnd(rng.standard_normal(shape), tc)
    g = (rng.standard_normal(pshape) * 0.1 + 1).astype(np.float32)
    b = (rng.standard_normal(pshape) * 0.1).astype(np.float32)
    f = B.LayerNormalization(B.context(type_config=tc), batch_axis=list(batch_axis), eps=1e-5)
    vx, vb, vg = var(x, half), var(b), var(g)
    vy, om, ov = B.Variable(shape), B.Variable(()), B.Variable(())
    f.setup([vx, vb, vg], [vy, om, ov])
    f.forward([vx, vb, vg], [vy, om, ov])
    y_r, m_r, v_r = R.ln_forward(x, b, g, outer, 1e-5)
    assert_close(vy.d, y_r, dn(tc), "y", "y")
    assert_close(om.d, m_r, dn(tc), "stat", "mean output")
    assert_close(ov.d, v_r, dn(tc), "stat", "var output")
    dm = rng.standard_normal(om.current_shape).astype(np.float32)
    dv = rng.standard_normal(ov.current_shape).astype(np.float32)
    vy.set_grad(dy, half)
    om.set_grad(dm)
    ov.set_grad(dv)
    pre = rng.standard_normal(shape).astype(np.float32)
    vx.set_grad(pre, half)
    f.backward([vx, vb, vg], [vy, om, ov], propagate_down=[1, 1, 1], accum=[1, 0, 0])
    dx_r, dg_r, db_r = R.ln_backward(x, dy, g, m_r, v_r, outer, 1e-5, dm, dv)
    assert_close(vx.g, dx_r + rnd(pre, tc), dn(tc), "grad", "dx accum with dmean/dvar")
    assert_close(vg.g, dg_r, dn(tc), "pgrad", "dgamma")
    assert_close(vb.g, db_r, dn(tc), "pgrad", "dbeta")


@pytest.mark.parametrize("tc", CONFIGS)
@pytest.mark.parametrize("shape,groups", [((4, 16, 8, 8), 4), ((2, 6, 5), 3), ((3, 8, 7, 7), 8)])
def test_group_normalization(tc, shape, groups):
    rng = np.random.default_rng(5)
    half = tc == "half"
    n, c = shape[0], shape[1]
    pshape = (1, c) + (1,) * (len(shape) - 2)
    x = rnd(rng.standard_normal(shape) * 1.5, tc)
    dy = rnd(rng.standard_normal(shape), tc)
    g = rng.uniform(0.5, 1.5, pshape).astype(np.float32)
    b = (rng.standard_normal(pshape) * 0.1).astype(np.float32)
    f = B.GroupNormalization(B.context(type_config=tc), num_groups=groups, channel_axis=1, batch_axis=[0])
    vx, vb, vg = var(x, half), var(b), var(g)
    vy = B.Variable(shape)
    f.setup([vx, vb, vg], [vy])
    f.forward([vx, vb, vg], [vy])
    y_r, m_r, v_r = R.gn_forward(x, b, g, n, c, groups, 1e-5)
    assert_close(vy.d, y_r, dn(tc), "y", "y")
    vy.set_grad(dy, half)
    f.backward([vx, vb, vg], [vy], propagate_down=[1, 1, 1], accum=[0, 0, 0])
    dx_r, dg_r, db_r = R.gn_backward(x, dy, g, m_r, v_r, n, c, groups, 1e-5)
    assert_close(vx.g, dx_r, dn(tc), "grad", "dx")
    assert_close(vg.g, dg_r, dn(tc), "pgrad", "dgamma")
    assert_close(vb.g, db_r, dn(tc), "pgrad", "dbeta")


@pytest.mark.parametrize("tc", CONFIGS)
@pytest.mark.parametrize("per_sample", [False, True])
def test_instance_normalization(tc, per_sample):
    rng = np.random.default_rng(6)
    half = tc == "half"
    shape = (3, 5, 9, 9)
    n, c = shape[0], shape[1]
    pshape = (n if per_sample else 1, c, 1, 1)
    x = rnd(rng.standard_normal(shape) * 1.5, tc)
    dy = rnd(rng.standard_normal(shape), tc)
    g = rng.uniform(0.5, 1.5, pshape).astype(np.float32)
    b = (rng.standard_normal(pshape) * 0.1).astype(np.float32)
    f = B.InstanceNormalization(B.context(type_config=tc), channel_axis=1, batch_axis=[0])
    vx, vb, vg = var(x, half), var(b), var(g)
    vy = B.Variable(shape)
    f.setup([vx, vb, vg], [vy])
    f.forward([vx, vb, vg], [vy])
    g_full = g.reshape(-1) if per_sample else np.tile(g.reshape(-1), n)
    b_full = b.reshape(-1) if per_sample else np.tile(b.reshape(-1), n)
    y_r, m_r, v_r = R.in_forward(x, b_full, g_full, n, c, 1e-5)
    assert_close(vy.d, y_r, dn(tc), "y", "y")
    vy.set_grad(dy, half)
    f.backward([vx, vb, vg], [vy], propagate_down=[1, 1, 1], accum=[0, 0, 0])
    dx_r, dg_r, db_r = R.in_backward(x, dy, g.reshape(-1), m_r, v_r, n, c, 1e-5,
                                     bc_gamma=not per_sample, bc_beta=not per_sample)
    assert_close(vx.g, dx_r, dn(tc), "grad", "dx")
    assert_close(vg.g, dg_r, dn(tc), "pgrad", "dgamma")
    assert_close(vb.g, db_r, dn(tc), "pgrad", "dbeta")


@pytest.mark.parametrize("tc", CONFIGS)
@pytest.mark.parametrize("shape,groups", [((4, 8, 8, 16), 4), ((2, 5, 6), 3), ((3, 7, 7, 24), 8)])
def test_group_normalization_channel_last(tc, shape, groups):
    """x[N, *spatial, C] with channel_axis = -1: no transposes, statistics as
    outputs [N, 1.., G], same numbers as the channel-first function on the
    transposed tensor (the reference's adaptor path, group_normalization.cu:93-106)."""
    rng = np.random.default_rng(8)
    half = tc == "half"
    n, c = shape[0], shape[-1]
    pshape = (1,) * (len(shape) - 1) + (c,)
    x = rnd(rng.standard_normal(shape) * 1.5, tc)
    dy = rnd(rng.standard_normal(shape), tc)
    g = rng.uniform(0.5, 1.5, pshape).astype(np.float32)
    b = (rng.standard_normal(pshape) * 0.1).astype(np.float32)
    f = B.GroupNormalization(B.context(type_config=tc), num_groups=groups, channel_axis=len(shape) - 1,
                             batch_axis=[0])
    vx, vb, vg = var(x, half), var(b), var(g)
    vy, om, ov = B.Variable(shape), B.Variable(()), B.Variable(())
    f.setup([vx, vb, vg], [vy, om, ov])
    assert tuple(om.current_shape) == (n,) + (1,) * (len(shape) - 2) + (groups,)
    f.forward([vx, vb, vg], [vy, om, ov])
    xt, dyt = np.moveaxis(x, -1, 1), np.moveaxis(dy, -1, 1)
    y_r, m_r, v_r = R.gn_forward(xt, b, g, n, c, groups, 1e-5)
    back = lambda a: np.moveaxis(np.asarray(a).reshape(xt.shape), 1, -1)
    assert_close(vy.d, back(y_r), dn(tc), "y", "y")
    assert_close(om.d, m_r, dn(tc), "stat", "mean output")
    assert_close(ov.d, v_r, dn(tc), "stat", "var output")
    dm = rng.standard_normal(om.current_shape).astype(np.float32)
    dv = rng.standard_normal(ov.current_shape).astype(np.float32)
    vy.set_grad(dy, half)
    om.set_grad(dm)
    ov.set_grad(dv)
    f.backward([vx, vb, vg], [vy, om, ov], propagate_down=[1, 1, 1], accum=[0, 0, 0])
    dx_r, dg_r, db_r = R.gn_backward(xt, dyt, g, m_r, v_r, n, c, groups, 1e-5, dm, dv)
    assert_close(vx.g, back(dx_r), dn(tc), "grad", "dx")
    assert_close(vg.g, dg_r, dn(tc), "pgrad", "dgamma")
    assert_close(vb.g, db_r, dn(tc), "pgrad", "dbeta")


@pytest.mark.parametrize("tc", CONFIGS)
@pytest.mark.parametrize("per_sample", [False, True])
def test_instance_normalization_channel_last(tc, per_sample):
    rng = np.random.default_rng(9)
    half = tc == "half"
    shape = (3, 9, 9, 8)
    n, c = shape[0], shape[-1]
    pshape = (n if per_sample else 1, 1, 1, c)
    x = rnd(rng.standard_normal(shape) * 1.5, tc)
    dy = rnd(rng.standard_normal(shape), tc)
    g = rng.uniform(0.5, 1.5, pshape).astype(np.float32)
    b = (rng.standard_normal(pshape) * 0.1).astype(np.float32)
    f = B.InstanceNormalization(B.context(type_config=tc), channel_axis=3, batch_axis=[0])
    vx, vb, vg = var(x, half), var(b), var(g)
    vy = B.Variable(shape)
    f.setup([vx, vb, vg], [vy])
    f.forward([vx, vb, vg], [vy])
    xt, dyt = np.moveaxis(x, -1, 1), np.moveaxis(dy, -1, 1)
    back = lambda a: np.moveaxis(np.asarray(a).reshape(xt.shape), 1, -1)
    g_full = g.reshape(-1) if per_sample else np.tile(g.reshape(-1), n)
    b_full = b.reshape(-1) if per_sample else np.tile(b.reshape(-1), n)
    y_r, m_r, v_r = R.in_forward(xt, b_full, g_full, n, c, 1e-5)
    assert_close(vy.d, back(y_r), dn(tc), "y", "y")
    vy.set_grad(dy, half)
    f.backward([vx, vb, vg], [vy], propagate_down=[1, 1, 1], accum=[0, 0, 0])
    dx_r, dg_r, db_r = R.in_backward(xt, dyt, g.reshape(-1), m_r, v_r, n, c, 1e-5,
                                     bc_gamma=not per_sample, bc_beta=not per_sample)
    assert_close(vx.g, back(dx_r), dn(tc), "grad", "dx")
    assert_close(vg.g, dg_r, dn(tc), "pgrad", "dgamma")
    assert_close(vb.g, db_r, dn(tc), "pgrad", "dbeta")


def test_group_count_must_divide_the_channels():
    ctx = B.context(type_config="float")
    x, y = B.Variable((4, 6, 8)), B.Variable((4, 6, 8))
    h = B.GroupNormalization(ctx, num_groups=4, channel_axis=1, batch_axis=[0], no_scale=True,
                             no_bias=True)
    with pytest.raises(B.NblaError, match="divisible"):
        h.setup([x], [y])


def test_extension_module_utilities():
    """The helpers the reference's Python package exports
    (python/src/nnabla_ext/cuda/__init__.py:124-160, init.pyx:74-205)."""
    assert B.array_classes()[0] == "HipCachedArray" and "HipArray" in B.array_classes()
    assert B.get_device_count() >= 1
    assert B.get_devices()[0] == "0"
    ctx = B.context(0, "half")
    assert ctx["backends"] == "hip:half,hip:float" and ctx["device_id"] == "0"
    assert B.context(device_id=0)["backends"] == "hip:float"
    with pytest.raises(ValueError):
        B.context(0, "mixed")
    B.synchronize(0)
    B.device_synchronize("0")
    B.clear_memory_cache()
    live, cached = B.memory_stats()
    assert cached == 0 and live >= 0


def test_pinned_host_array_class_gives_the_same_results():
    """Staging through HipCachedHostArray (page-locked memory) instead of
    CpuArray changes nothing but the transfer path."""
    rng = np.random.default_rng(23)
    x = rng.standard_normal((16, 8, 12, 12)).astype(np.float32)
    dy = rng.standard_normal(x.shape).astype(np.float32)

    def run():
        f = B.InstanceNormalization(B.context(type_config="half"), channel_axis=1, batch_axis=[0], no_scale=True,
                                    no_bias=True)
        vx, vy = var(x, True), B.Variable(x.shape)
        f.setup([vx], [vy])
        f.forward([vx], [vy])
        vy.set_grad(dy, True)
        f.backward([vx], [vy], propagate_down=[1], accum=[0])
        return vy.d.copy(), vx.g.copy()

    y0, dx0 = run()
    B.set_host_array_class("HipCachedHostArray")
    try:
        y1, dx1 = run()
    finally:
        B.set_host_array_class("CpuArray")
    np.testing.assert_array_equal(y0, y1)
    np.testing.assert_array_equal(dx0, dx1)
    with pytest.raises(B.NblaError, match="host array class"):
        B.set_host_array_class("NoSuchArray")


def test_caching_allocator_reuses_blocks():
    import ctypes
    L = B.lib()
    live, cached = ctypes.c_uint64(), ctypes.c_uint64()
    ctx = B.context(type_config="float")
    x = np.random.default_rng(7).standard_normal((64, 256)).astype(np.float32)

    def run():
        f = B.LayerNormalization(ctx, batch_axis=[0], no_scale=True, no_bias=True)
        vx, vy = var(x), B.Variable(x.shape)
        f.setup([vx], [vy])
        f.forward([vx], [vy])
        return vy.d

    a = run()
    L.nnabla_hip_memory_stats(ctypes.byref(live), ctypes.byref(cached))
    assert cached.value > 0                      # freed arrays went to the cache
    c1 = cached.value
    b = run()
    np.testing.assert_array_equal(a, b)
    L.nnabla_hip_memory_stats(ctypes.byref(live), ctypes.byref(cached))
    assert cached.value == c1                    # second run was served from it
    assert L.nnabla_hip_clear_memory_cache() == 0
    L.nnabla_hip_memory_stats(ctypes.byref(live), ctypes.byref(cached))
    assert cached.value == 0


def _tensor_norm_reference(x, dy, g, b, keep, eps, dm=None, dv=None):
    """float64 torch autograd of y = (x - mean) / sqrt(var + eps) * g + b with
    statistics over every axis not in `keep` (biased variance)."""
    red = [i for i in range(x.ndim) if i not in keep]
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    gt = None if g is None else torch.tensor(g, dtype=torch.float64, requires_grad=True)
    bt = None if b is None else torch.tensor(b, dtype=torch.float64, requires_grad=True)
    m = xt.mean(red, keepdim=True)
    v = xt.var(red, unbiased=False, keepdim=True)
    y = (xt - m) / torch.sqrt(v + eps)
    if gt is not None:
        y = y * gt
    if bt is not None:
        y = y + bt
    loss = (y * torch.tensor(dy, dtype=torch.float64)).sum()
    if dm is not None:
        loss = loss + (m * torch.tensor(dm, dtype=torch.float64)).sum()
        loss = loss + (v * torch.tensor(dv, dtype=torch.float64)).sum()
    loss.backward()
    out = lambda t: None if t is None else t.grad.numpy()
    return (y.detach().numpy(), m.detach().numpy(), v.detach().numpy(), xt.grad.numpy(), out(gt),
            out(bt))


@pytest.mark.parametrize("tc", CONFIGS)
@pytest.mark.parametrize("shape,axes", [((4, 6, 5, 8), [1]), ((4, 6, 5, 8), [0, 1]),
                                        ((4, 6, 5, 8), [3]), ((4, 6, 5, 8), [2, 3]),
                                        ((4, 6, 5, 8), [1, 2]), ((3, 40, 14, 14), [-3]),
                                        ((64, 48), [0]), ((2, 3, 4, 5, 6), [1, 2, 3]),
                                        ((4, 6, 5, 8), [0, 2]), ((4, 6, 5, 8), [1, 3]),
                                        ((4, 6, 5, 8), [0, 3]), ((2, 3, 4, 5, 6), [0, 2, 4]),
                                        ((3, 70, 9, 66), [1, 3])])
def test_tensor_normalization(tc, shape, axes):
    """TensorNormalization over adjacent kept axes (read in place) and over
    other sets (gathered by a device permutation) against float64 autograd of
    the defining formula; statistics as outputs with gradients flowing into
    them."""
    rng = np.random.default_rng(21)
    half = tc == "half"
    keep = sorted(a % len(shape) for a in axes)
    pshape = tuple(s if i in keep else 1 for i, s in enumerate(shape))
    x = rnd(rng.standard_normal(shape) * 1.5 + 0.5, tc)
    dy = rnd(rng.standard_normal(shape), tc)
    g = rng.uniform(0.5, 1.5, pshape).astype(np.float32)
    b = (rng.standard_normal(pshape) * 0.1).astype(np.float32)
    dm = rng.standard_normal(pshape).astype(np.float32)
    dv = rng.standard_normal(pshape).astype(np.float32)
    f = B.TensorNormalization(B.context(type_config=tc), axes=axes, eps=1e-5)
    assert f.name == "TensorNormalizationHip"
    vx, vb, vg = var(x, half), var(b), var(g)
    vy, om, ov = B.Variable(shape), B.Variable(()), B.Variable(())
    f.setup([vx, vb, vg], [vy, om, ov])
    assert om.current_shape == pshape and ov.current_shape == pshape
    f.forward([vx, vb, vg], [vy, om, ov])
    y_r, m_r, v_r, dx_r, dg_r, db_r = _tensor_norm_reference(x, dy, g, b, keep, 1e-5, dm, dv)
    assert_close(vy.d, y_r, dn(tc), "y", "y")
    assert_close(om.d, m_r, dn(tc), "stat", "mean")
    assert_close(ov.d, v_r, dn(tc), "stat", "var")
    vy.set_grad(dy, half)
    om.set_grad(dm)
    ov.set_grad(dv)
    f.backward([vx, vb, vg], [vy, om, ov], propagate_down=[1, 1, 1], accum=[0, 0, 0])
    assert_close(vx.g, dx_r, dn(tc), "grad", "dx")
    assert_close(vg.g, dg_r, dn(tc), "pgrad", "dgamma")
    assert_close(vb.g, db_r, dn(tc), "pgrad", "dbeta")
    # one output, no scale / no bias, accumulation onto dx
    f1 = B.TensorNormalization(B.context(type_config=tc), axes=axes, eps=1e-5, no_scale=True,
                               no_bias=True)
    vy1 = B.Variable(shape)
    f1.setup([vx], [vy1])
    f1.forward([vx], [vy1])
    y1, _, _, dx1, _, _ = _tensor_norm_reference(x, dy, None, None, keep, 1e-5)
    assert_close(vy1.d, y1, dn(tc), "y", "y plain")
    pre = rnd(rng.standard_normal(shape), tc)
    vx.set_grad(pre, half)
    vy1.set_grad(dy, half)
    f1.backward([vx], [vy1], propagate_down=[1], accum=[1])
    assert_close(vx.g, dx1 + pre, dn(tc), "grad", "dx accumulated")


@pytest.mark.parametrize("tc", CONFIGS)
@pytest.mark.parametrize("shape,axis", [((16, 8, 3, 3), 0), ((8, 16, 3, 3), 1), ((64, 576), 0),
                                        ((3, 3, 8, 32), -1)])
def test_weight_standardization(tc, shape, axis):
    rng = np.random.default_rng(22)
    half = tc == "half"
    keep = [axis % len(shape)]
    pshape = tuple(s if i in keep else 1 for i, s in enumerate(shape))
    w = rnd(rng.standard_normal(shape) * 0.2 + 0.05, tc)
    dy = rnd(rng.standard_normal(shape), tc)
    f = B.WeightStandardization(B.context(type_config=tc), channel_axis=axis, eps=1e-5)
    assert f.name == "WeightStandardizationHip"
    vw, vy = var(w, half), B.Variable(shape)
    f.setup([vw], [vy])
    f.forward([vw], [vy])
    y_r, m_r, v_r, dw_r, _, _ = _tensor_norm_reference(w, dy, None, None, keep, 1e-5)
    assert_close(vy.d, y_r, dn(tc), "y", "y")
    vy.set_grad(dy, half)
    f.backward([vw], [vy], propagate_down=[1], accum=[0])
    assert_close(vw.g, dw_r, dn(tc), "grad", "dw")
    # statistics as outputs
    om, ov = B.Variable(()), B.Variable(())
    f.setup([vw], [vy, om, ov])
    f.forward([vw], [vy, om, ov])
    assert om.current_shape == pshape
    assert_close(om.d, m_r, dn(tc), "stat", "mean")
    assert_close(ov.d, v_r, dn(tc), "stat", "var")


def test_tensor_normalization_argument_errors():
    ctx = B.context(type_config="float")
    x, y = B.Variable((4, 6, 5, 8)), B.Variable((4, 6, 5, 8))
    with pytest.raises(RuntimeError, match="out of range"):
        B.TensorNormalization(ctx, axes=[4], no_scale=True, no_bias=True).setup([x], [y])
    with pytest.raises(RuntimeError, match="elements"):
        B.TensorNormalization(ctx, axes=[1], no_scale=True).setup([x, B.Variable((1, 5, 1, 1))], [y])
    with pytest.raises(RuntimeError, match="out of range"):
        B.WeightStandardization(ctx, channel_axis=7).setup([x], [y])
