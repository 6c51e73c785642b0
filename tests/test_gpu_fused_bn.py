"""FusedBatchNormalization (BatchNormalization + residual add + ReLU) parity on
the GPU: the HIP path through the C-ABI against the float64 oracle.

The backward gates dy by the sign of the stored forward output
(include/nbla/cuda/utils/relu.cuh:56-62), so both sides are given the SAME y
(the one the GPU forward produced): an element whose pre-activation rounds to
zero on one side only would otherwise flip its gate."""
import numpy as np
import pytest
import torch

from _util import assert_close, dtype_name, load_package, rounded, to_dev, to_np
from oracle import norm_ref as R

pytestmark = pytest.mark.gpu
K = load_package()
DTYPES = [torch.float32, torch.float16]

# (shape, axis): planes layout, channel-last (register-resident parameters and
# the generic apply), odd sizes (scalar loads), one channel, 2-D input, enough
# channels for the channel-owning reduction blocks.
SHAPES = [
    ((4, 8, 6, 6), 1), ((2, 3, 5, 7), 1), ((3, 16, 49), 1), ((5, 7), 1), ((2, 1, 9), 1),
    ((6, 5, 4, 8), 3), ((64, 64), 1), ((7, 3, 5, 12), 3), ((129, 5, 5, 96), 3),
    ((3, 2, 2, 2050), 3), ((2, 256, 9, 9), 1), ((8, 14, 14, 64), 3),
    ((8, 12, 14, 14), 1), ((16, 256, 14, 14), 1),
    ((4, 8, 7, 7), 1), ((64, 32, 7, 7), 1), ((5, 16, 13), 1),
    ((6, 9, 9, 96), 3), ((3, 5, 5, 4104), 3), ((37, 100), 1),
    # channel-last with few rows: a channel vector's column in one block's registers
    ((32, 7, 7, 512), 3), ((8, 14, 14, 256), 3), ((100, 2048), 1), ((33, 8, 8, 320), 3),
    # planes layout with a channel held on one CU in the forward (registers, then LDS;
    # the last one with a streamed remainder)
    ((36, 64, 32, 32), 1), ((73, 48, 32, 32), 1), ((230, 232, 16, 32), 1),
]


def make(shape, axis, dtype, seed, with_z=True):
    rng = np.random.default_rng(seed)
    c = shape[axis]
    x = rounded(rng.standard_normal(shape) * 2.0 + 1.0, dtype)
    z = rounded(rng.standard_normal(shape), dtype) if with_z else None
    dy = rounded(rng.standard_normal(shape), dtype)
    g = rng.uniform(0.5, 1.5, c).astype(np.float32).astype(np.float64)
    b = (rng.standard_normal(c) * 0.3).astype(np.float32).astype(np.float64)
    rm = (rng.standard_normal(c) * 0.1 + 1.0).astype(np.float32).astype(np.float64)
    rv = rng.uniform(2.0, 6.0, c).astype(np.float32).astype(np.float64)
    return x, z, dy, g, b, rm, rv


@pytest.mark.parametrize("shape,axis", SHAPES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("with_z", [True, False])
def test_fused_bn_training(shape, axis, dtype, with_z):
    c = shape[axis]
    if int(np.prod(shape)) // c < 2:
        pytest.skip("N == 1")
    dn = dtype_name(dtype)
    x, z, dy, g, b, rm, rv = make(shape, axis, dtype, 41, with_z)
    y_r, m_r, v_r, rm_r, rv_r = R.fused_bn_forward(x, z, b, g, rm, rv, axis, 0.9, 1e-5, True)
    xd, dyd, gd, bd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(b)
    zd = to_dev(z, dtype) if with_z else None
    rmd, rvd = to_dev(rm), to_dev(rv)
    y, m, v = K.fused_bn_forward_batch(xd, zd, bd, gd, rmd, rvd, axis, 0.9, 1e-5)
    assert_close(to_np(y), y_r, dn, "y", "y")
    assert (to_np(y) >= 0).all()
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(rmd), rm_r, dn, "stat", "running_mean")
    assert_close(to_np(rvd), rv_r, dn, "stat", "running_var")
    y_gpu = to_np(y).astype(np.float64)
    dx_r, dz_r, dg_r, db_r = R.fused_bn_backward(x, y_gpu, dy, g, m_r, v_r, axis, 1e-5, True)
    dx, dz, dg, db = K.fused_bn_backward(xd, y, dyd, gd, m, v, axis, 1e-5)
    assert_close(to_np(dx), dx_r, dn, "grad", "dx")
    np.testing.assert_array_equal(to_np(dz).astype(np.float64), dz_r)   # a gated copy: exact
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


@pytest.mark.parametrize("shape,axis", [((4, 8, 6, 6), 1), ((6, 5, 4, 8), 3), ((33, 24), 1)])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("with_z", [True, False])
def test_fused_bn_inference_mode(shape, axis, dtype, with_z):
    dn = dtype_name(dtype)
    x, z, dy, g, b, rm, rv = make(shape, axis, dtype, 42, with_z)
    y_r, _, _, _, _ = R.fused_bn_forward(x, z, b, g, rm, rv, axis, 0.9, 1e-5, False)
    xd, dyd, gd, bd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(b)
    zd = to_dev(z, dtype) if with_z else None
    rmd, rvd = to_dev(rm), to_dev(rv)
    y = K.fused_bn_forward_global(xd, zd, bd, gd, rmd, rvd, axis, 1e-5)
    assert_close(to_np(y), y_r, dn, "y", "y")
    np.testing.assert_array_equal(to_np(rmd), rm.astype(np.float32))   # read-only here
    y_gpu = to_np(y).astype(np.float64)
    dx_r, dz_r, dg_r, db_r = R.fused_bn_backward(x, y_gpu, dy, g, rm, rv, axis, 1e-5, False)
    dx, dz, dg, db = K.fused_bn_backward(xd, y, dyd, gd, rmd, rvd, axis, 1e-5, batch_stat=False)
    assert_close(to_np(dx), dx_r, dn, "grad", "dx")
    np.testing.assert_array_equal(to_np(dz).astype(np.float64), dz_r)
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


@pytest.mark.parametrize("shape,axis", [((4, 8, 6, 6), 1), ((6, 5, 4, 8), 3), ((37, 24), 1)])
def test_fused_bn_flags(shape, axis):
    """3-output dmean/dvar, accumulation onto dx/dz/dgamma/dbeta,
    propagate_down subsets (dz only, dx only, parameters only), dz written in
    place of dy."""
    c = shape[axis]
    x, z, dy, g, b, rm, rv = make(shape, axis, torch.float32, 43)
    rng = np.random.default_rng(44)
    dm, dv = rng.standard_normal(c), rng.standard_normal(c)
    xd, zd, dyd, gd, bd = to_dev(x), to_dev(z), to_dev(dy), to_dev(g), to_dev(b)
    y, m, v = K.fused_bn_forward_batch(xd, zd, bd, gd, None, None, axis, 0.9, 1e-5)
    y_gpu = to_np(y).astype(np.float64)
    _, m_r, v_r, _, _ = R.fused_bn_forward(x, z, b, g, None, None, axis, 0.9, 1e-5, True)
    dx_r, dz_r, dg_r, db_r = R.fused_bn_backward(x, y_gpu, dy, g, m_r, v_r, axis, 1e-5, True, dm, dv)

    pre_dx = rng.standard_normal(shape).astype(np.float32)
    pre_dz = rng.standard_normal(shape).astype(np.float32)
    pre_g = rng.standard_normal(c).astype(np.float32)
    pre_b = rng.standard_normal(c).astype(np.float32)
    dxd, dzd, dgd, dbd = to_dev(pre_dx), to_dev(pre_dz), to_dev(pre_g), to_dev(pre_b)
    K.fused_bn_backward(xd, y, dyd, gd, m, v, axis, 1e-5, dmean=to_dev(dm), dvar=to_dev(dv),
                        dx=dxd, dz=dzd, dgamma=dgd, dbeta=dbd, accum=(True, True, True, True))
    assert_close(to_np(dxd), dx_r + pre_dx, "f32", "grad", "dx accum 3-output")
    assert_close(to_np(dzd), dz_r + pre_dz, "f32", "grad", "dz accum")
    assert_close(to_np(dgd), dg_r + pre_g, "f32", "pgrad", "dgamma accum")
    assert_close(to_np(dbd), db_r + pre_b, "f32", "pgrad", "dbeta accum")

    dx_r, dz_r, dg_r, db_r = R.fused_bn_backward(x, y_gpu, dy, g, m_r, v_r, axis, 1e-5, True)
    _, dz, _, _ = K.fused_bn_backward(xd, y, dyd, gd, m, v, axis, 1e-5,
                                      need=(False, True, False, False))
    np.testing.assert_array_equal(to_np(dz).astype(np.float64), dz_r)
    dx, _, _, _ = K.fused_bn_backward(xd, y, dyd, gd, m, v, axis, 1e-5,
                                      need=(True, False, False, False))
    assert_close(to_np(dx), dx_r, "f32", "grad", "dx only")
    _, _, dg, db = K.fused_bn_backward(xd, y, dyd, gd, m, v, axis, 1e-5,
                                       need=(False, False, True, True))
    assert_close(to_np(dg), dg_r, "f32", "pgrad", "dgamma only")
    assert_close(to_np(db), db_r, "f32", "pgrad", "dbeta only")
    # dz aliasing dy: every element is read before it is overwritten
    dy_copy = dyd.clone()
    dx, dz, dg, db = K.fused_bn_backward(xd, y, dy_copy, gd, m, v, axis, 1e-5, dz=dy_copy)
    assert_close(to_np(dx), dx_r, "f32", "grad", "dx, dz in place of dy")
    np.testing.assert_array_equal(to_np(dy_copy).astype(np.float64), dz_r)
    assert_close(to_np(dg), dg_r, "f32", "pgrad", "dgamma, dz in place of dy")


def test_fused_bn_gate_follows_stored_output():
    """The gate is y > 0 on the stored output: -0.0, +0.0 and negative values
    close it, any positive value (denormal, inf) opens it."""
    for dtype in DTYPES:
        vals = torch.tensor([0.0, -0.0, 1e-7 if dtype == torch.float32 else 6e-8, 1.0, -1.0,
                             float("inf"), -float("inf"), 65504.0], dtype=dtype, device="cuda")
        y = vals.repeat(64).reshape(8, 8, 8).contiguous()          # [N, C, S]
        x = torch.randn_like(y)
        dy = torch.ones_like(y) * 3
        m = torch.zeros(8, device="cuda")
        v = torch.ones(8, device="cuda")
        _, dz, _, _ = K.fused_bn_backward(x, y, dy, None, m, v, 1, 1e-5, batch_stat=False)
        want = torch.where(y > 0, dy, torch.zeros_like(dy))
        assert torch.equal(dz, want)


def test_fused_bn_resnet_block_full_size():
    """ResNet-50 stage-2 activation stored NHWC, fp16: x, z [32,56,56,256]."""
    shape, axis, dtype = (32, 56, 56, 256), 3, torch.float16
    rng = np.random.default_rng(45)
    c = shape[axis]
    x = (rng.standard_normal(shape, dtype=np.float32) * 2 + 1).astype(np.float16)
    z = rng.standard_normal(shape, dtype=np.float32).astype(np.float16)
    dy = rng.standard_normal(shape, dtype=np.float32).astype(np.float16)
    g = rng.uniform(0.5, 1.5, c).astype(np.float32)
    b = (rng.standard_normal(c) * 0.3).astype(np.float32)
    xd, zd, dyd = torch.from_numpy(x).cuda(), torch.from_numpy(z).cuda(), torch.from_numpy(dy).cuda()
    gd, bd = to_dev(g), to_dev(b)
    rmd, rvd = torch.zeros(c, device="cuda"), torch.ones(c, device="cuda")
    y, m, v = K.fused_bn_forward_batch(xd, zd, bd, gd, rmd, rvd, axis, 0.9, 1e-5)
    dx, dz, dg, db = K.fused_bn_backward(xd, y, dyd, gd, m, v, axis, 1e-5)
    y_r, m_r, v_r, rm_r, rv_r = R.fused_bn_forward(x, z, b, g, np.zeros(c), np.ones(c), axis, 0.9,
                                                   1e-5, True)
    assert_close(to_np(y), y_r, "f16", "y", "y")
    assert_close(to_np(m), m_r, "f16", "stat", "mean")
    assert_close(to_np(v), v_r, "f16", "stat", "var")
    assert_close(to_np(rvd), rv_r, "f16", "stat", "running_var")
    y_gpu = to_np(y)
    dx_r, dz_r, dg_r, db_r = R.fused_bn_backward(x, y_gpu, dy, g, m_r, v_r, axis, 1e-5, True)
    assert_close(to_np(dx), dx_r, "f16", "grad", "dx")
    assert np.array_equal(to_np(dz), dz_r.astype(np.float16))
    assert_close(to_np(dg), dg_r, "f16", "pgrad", "dgamma")
    assert_close(to_np(db), db_r, "f16", "pgrad", "dbeta")
    # determinism
    y2, m2, v2 = K.fused_bn_forward_batch(xd, zd, bd, gd, None, None, axis, 0.9, 1e-5)
    dx2, dz2, dg2, db2 = K.fused_bn_backward(xd, y2, dyd, gd, m2, v2, axis, 1e-5)
    for a, c2 in ((y, y2), (m, m2), (dx, dx2), (dz, dz2), (dg, dg2), (db, db2)):
        assert torch.equal(a, c2)


def test_fused_bn_argument_errors():
    L = K.lib()
    s = torch.cuda.current_stream().cuda_stream
    x = torch.randn(4, 8, 16, device="cuda")
    y = torch.empty_like(x)
    m = torch.zeros(8, device="cuda")
    ws = torch.empty(max(1, L.nblahip_bn_workspace_bytes(4, 8, 16, 0)), dtype=torch.uint8,
                     device="cuda")
    args = (4, 8, 16, 1e-5, 1, 0, ws.data_ptr(), ws.numel(), s)
    # the forward output is required
    assert L.nblahip_fused_bn_bwd(x.data_ptr(), None, x.data_ptr(), None, m.data_ptr(),
                                  m.data_ptr(), None, None, y.data_ptr(), None, None, None, 0, 0,
                                  0, 0, *args) == -1
    # workspace missing
    assert L.nblahip_fused_bn_bwd(x.data_ptr(), y.data_ptr(), x.data_ptr(), None, m.data_ptr(),
                                  m.data_ptr(), None, None, y.data_ptr(), None, None, None, 0, 0,
                                  0, 0, 4, 8, 16, 1e-5, 1, 0, None, 0, s) == -2
    # empty tensor: no-op
    assert L.nblahip_fused_bn_fwd_infer(None, None, None, None, None, None, None, 0, 8, 16, 1e-5,
                                        0, s) == 0
