"""Parameters and statistics that a "hip:half" graph stores in half precision
(the reference's plain cuda:half type config keeps gamma, beta, mean, var,
running statistics and their gradients in Tc = half:
layer_normalization.cu:91-93, batch_normalization.cu:124-143).  The Function
classes read and write such arrays where they lie (one staging launch each
way around the float32-parameter kernels): results must match the oracle fed
with the half-rounded parameters, at the fp16 tolerances, and every array must
keep the type it is stored in - the running statistics and the accumulated
gradients above all.  Arrays stored as float stay float (the other test files
cover those)."""
import numpy as np
import pytest

from _util import assert_close, load_package
from oracle import norm_ref as R

load_package()
from nnabla_ext_cuda_amd import binding as B  # noqa: E402

pytestmark = pytest.mark.gpu


def h(a):
    """Half-rounded copy as float64 (what the oracle sees)."""
    return np.asarray(a, np.float32).astype(np.float16).astype(np.float64)


def var(a, half=True):
    v = B.Variable(np.shape(a))
    v.set_data(a, half=half)
    return v


@pytest.fixture(scope="module", autouse=True)
def _init():
    B.init()


def ctx():
    return B.context(type_config="half")


@pytest.mark.parametrize("shape,axis", [((4, 8, 6, 6), 1), ((6, 5, 4, 8), 3)])
def test_batch_normalization_keeps_half_parameters_and_running_statistics(shape, axis):
    rng = np.random.default_rng(11)
    c = shape[axis]
    pshape = tuple(c if i == axis else 1 for i in range(len(shape)))
    x, dy = h(rng.standard_normal(shape) * 2 + 1), h(rng.standard_normal(shape))
    g, b = h(rng.uniform(0.5, 1.5, pshape)), h(rng.standard_normal(pshape) * 0.1)
    rm, rv = h(rng.standard_normal(pshape) * 0.1), h(rng.uniform(0.5, 2, pshape))
    f = B.BatchNormalization(ctx(), axes=[axis], decay_rate=0.9, eps=1e-5, batch_stat=True)
    vx, vb, vg, vm, vv = var(x), var(b), var(g), var(rm), var(rv)
    vy, om, ov = B.Variable(shape), B.Variable(()), B.Variable(())
    ins, outs = [vx, vb, vg, vm, vv], [vy, om, ov]
    f.setup(ins, outs)
    f.forward(ins, outs)
    y_r, m_r, v_r, rm_r, rv_r = R.bn_forward_batch(x, b, g, rm, rv, axis, 0.9, 1e-5)
    assert_close(vy.d, y_r, "f16", "y", "y")
    # stored types: parameters untouched, running statistics and exposed statistics half
    assert [v.stored_dtype() for v in (vb, vg, vm, vv, om, ov)] == ["half"] * 6
    assert_close(vm.d, h(rm_r), "f16", "y", "running mean, stored in half")
    assert_close(vv.d, h(rv_r), "f16", "y", "running var, stored in half")
    assert_close(om.d, h(m_r), "f16", "y", "mean output")
    assert_close(ov.d, h(v_r), "f16", "y", "var output")
    # backward reads the half statistics it exposed and their gradients
    dm, dv = h(rng.standard_normal(om.current_shape)), h(rng.standard_normal(ov.current_shape))
    vy.set_grad(dy, True)
    om.set_grad(dm, True)
    ov.set_grad(dv, True)
    f.backward(ins, outs, propagate_down=[1, 1, 1, 0, 0], accum=[0, 0, 0, 0, 0])
    dx_r, dg_r, db_r = R.bn_backward_batch(x, dy, g, om.d.astype(np.float64), ov.d.astype(np.float64),
                                           axis, 1e-5, dm, dv)
    assert_close(vx.g, dx_r, "f16", "grad", "dx")
    assert vg.stored_dtype(1) == "half" and vb.stored_dtype(1) == "half"
    assert_close(vg.g, dg_r, "f16", "grad", "dgamma, stored in half")
    assert_close(vb.g, db_r, "f16", "grad", "dbeta, stored in half")
    # accumulation onto the half gradients keeps them half
    f.backward(ins, outs, propagate_down=[0, 1, 1, 0, 0], accum=[0, 1, 1, 0, 0])
    assert vg.stored_dtype(1) == "half" and vb.stored_dtype(1) == "half"
    assert_close(vg.g, 2 * dg_r, "f16", "grad", "dgamma accumulated")
    # inference with the (half) running statistics
    fi = B.BatchNormalization(ctx(), axes=[axis], decay_rate=0.9, eps=1e-5, batch_stat=False)
    vy2 = B.Variable(shape)
    fi.setup(ins, [vy2])
    fi.forward(ins, [vy2])
    y_i = R.bn_forward_global(x, b, g, vm.d.astype(np.float64), vv.d.astype(np.float64), axis, 1e-5)
    assert_close(vy2.d, y_i, "f16", "y", "inference y")
    assert vm.stored_dtype() == "half" and vv.stored_dtype() == "half"


def test_mixed_storage_is_read_as_it_lies():
    """gamma in half, beta and the running statistics in float: each keeps its type."""
    rng = np.random.default_rng(12)
    shape, axis, c = (8, 16, 5, 5), 1, 16
    pshape = (1, c, 1, 1)
    x = h(rng.standard_normal(shape) + 0.5)
    g = h(rng.uniform(0.5, 1.5, pshape))
    b = (rng.standard_normal(pshape) * 0.1).astype(np.float32).astype(np.float64)
    rm, rv = np.zeros(pshape), np.ones(pshape)
    f = B.BatchNormalization(ctx(), axes=[axis], decay_rate=0.9, eps=1e-5, batch_stat=True)
    vx, vb, vg, vm, vv = var(x), var(b, half=False), var(g), var(rm, half=False), var(rv, half=False)
    vy = B.Variable(shape)
    f.setup([vx, vb, vg, vm, vv], [vy])
    f.forward([vx, vb, vg, vm, vv], [vy])
    y_r, _, _, rm_r, rv_r = R.bn_forward_batch(x, b, g, rm, rv, axis, 0.9, 1e-5)
    assert_close(vy.d, y_r, "f16", "y", "y")
    assert [v.stored_dtype() for v in (vb, vg, vm, vv)] == ["float", "half", "float", "float"]
    assert_close(vm.d, rm_r, "f16", "stat", "running mean stays float32")
    assert_close(vv.d, rv_r, "f16", "stat", "running var stays float32")


def test_layer_normalization_half_parameters():
    rng = np.random.default_rng(13)
    shape, outer = (6, 10, 256), 60
    pshape = (1, 1, 256)
    x, dy = h(rng.standard_normal(shape) + 2), h(rng.standard_normal(shape))
    g, b = h(rng.standard_normal(pshape) * 0.1 + 1), h(rng.standard_normal(pshape) * 0.1)
    f = B.LayerNormalization(ctx(), batch_axis=[0, 1], eps=1e-5)
    vx, vb, vg = var(x), var(b), var(g)
    vy, om, ov = B.Variable(shape), B.Variable(()), B.Variable(())
    f.setup([vx, vb, vg], [vy, om, ov])
    f.forward([vx, vb, vg], [vy, om, ov])
    y_r, m_r, v_r = R.ln_forward(x, b, g, outer, 1e-5)
    assert_close(vy.d, y_r, "f16", "y", "y")
    assert [v.stored_dtype() for v in (vb, vg, om, ov)] == ["half"] * 4
    assert_close(om.d, h(m_r), "f16", "y", "mean output")
    assert_close(ov.d, h(v_r), "f16", "y", "var output")
    vy.set_grad(dy, True)
    om.zero_grad()
    ov.zero_grad()
    f.backward([vx, vb, vg], [vy, om, ov], propagate_down=[1, 1, 1], accum=[0, 0, 0])
    dx_r, dg_r, db_r = R.ln_backward(x, dy, g, om.d.astype(np.float64).ravel(),
                                     ov.d.astype(np.float64).ravel(), outer, 1e-5)
    assert_close(vx.g, dx_r, "f16", "grad", "dx")
    assert vg.stored_dtype(1) == "half" and vb.stored_dtype(1) == "half"
    assert_close(vg.g, dg_r, "f16", "grad", "dgamma")
    assert_close(vb.g, db_r, "f16", "grad", "dbeta")


@pytest.mark.parametrize("kind,cl", [("gn", False), ("gn", True), ("in", False), ("in", True)])
def test_group_and_instance_normalization_half_parameters(kind, cl):
    rng = np.random.default_rng(14)
    n, c, sp, groups = 3, 64, (6, 6), 8
    shape = (n,) + sp + (c,) if cl else (n, c) + sp
    caxis = len(shape) - 1 if cl else 1
    pshape = tuple(c if i == caxis else 1 for i in range(len(shape)))
    x, dy = h(rng.standard_normal(shape) * 1.5), h(rng.standard_normal(shape))
    g, b = h(rng.uniform(0.5, 1.5, pshape)), h(rng.standard_normal(pshape) * 0.1)
    if kind == "gn":
        f = B.GroupNormalization(ctx(), num_groups=groups, channel_axis=caxis, batch_axis=[0], eps=1e-5)
    else:
        f = B.InstanceNormalization(ctx(), channel_axis=caxis, batch_axis=[0], eps=1e-5)
    vx, vb, vg = var(x), var(b), var(g)
    vy = B.Variable(shape)
    f.setup([vx, vb, vg], [vy])
    f.forward([vx, vb, vg], [vy])
    xt = np.moveaxis(x, -1, 1) if cl else x
    dyt = np.moveaxis(dy, -1, 1) if cl else dy
    back = (lambda a: np.moveaxis(np.asarray(a).reshape(xt.shape), 1, -1)) if cl else \
        (lambda a: np.asarray(a).reshape(xt.shape))
    if kind == "gn":
        y_r, m_r, v_r = R.gn_forward(xt, b.ravel(), g.ravel(), n, c, groups, 1e-5)
        dx_r, dg_r, db_r = R.gn_backward(xt, dyt, g.ravel(), m_r, v_r, n, c, groups, 1e-5)
    else:
        y_r, m_r, v_r = R.in_forward(xt, b.ravel(), g.ravel(), n, c, 1e-5)
        dx_r, dg_r, db_r = R.in_backward(xt, dyt, g.ravel(), m_r, v_r, n, c, 1e-5)
    assert_close(vy.d, back(y_r), "f16", "y", "y")
    vy.set_grad(dy, True)
    f.backward([vx, vb, vg], [vy], propagate_down=[1, 1, 1], accum=[0, 0, 0])
    assert_close(vx.g, back(dx_r), "f16", "grad", "dx")
    assert [vb.stored_dtype(), vg.stored_dtype(), vb.stored_dtype(1), vg.stored_dtype(1)] == ["half"] * 4
    assert_close(vg.g.ravel(), dg_r, "f16", "grad", "dgamma")
    assert_close(vb.g.ravel(), db_r, "f16", "grad", "dbeta")


def test_stage_params_entry_point():
    """nblahip_stage_params: several arrays, one launch each way, bit-exact
    float16 <-> float32 conversion; argument errors."""
    import ctypes

    import torch
    K = load_package()
    L = K.lib()
    s = torch.cuda.current_stream().cuda_stream
    sizes = [1, 7, 64, 1000, 0, 5000]
    srcs = [torch.randn(max(n, 1), device="cuda").half() for n in sizes]
    dsts = [torch.zeros(max(n, 1), device="cuda") for n in sizes]
    P = ctypes.c_void_p * len(sizes)
    N = ctypes.c_int64 * len(sizes)
    K.check(L.nblahip_stage_params(len(sizes), P(*[t.data_ptr() for t in srcs]), K.F16,
                                   P(*[t.data_ptr() for t in dsts]), K.F32, N(*sizes), s))
    for n, a, b_ in zip(sizes, srcs, dsts):
        assert torch.equal(b_[:n], a[:n].float())
    back = [torch.zeros(max(n, 1), device="cuda").half() for n in sizes]
    K.check(L.nblahip_stage_params(len(sizes), P(*[t.data_ptr() for t in dsts]), K.F32,
                                   P(*[t.data_ptr() for t in back]), K.F16, N(*sizes), s))
    for n, a, b_ in zip(sizes, srcs, back):
        assert torch.equal(b_[:n], a[:n])
    assert L.nblahip_stage_params(17, P(), K.F16, P(), K.F32, N(), s) == -1
    assert L.nblahip_stage_params(1, P(), K.F32, P(), K.F32, N(), s) == -1
    assert L.nblahip_stage_params(0, None, K.F16, None, K.F32, None, s) == 0
