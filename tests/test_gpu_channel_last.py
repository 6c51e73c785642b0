"""Channel-last GroupNormalization / InstanceNormalization on the GPU: the HIP
path through the C-ABI on x[N, *spatial, C] against the float64 oracle applied
to the channel-first transpose (what the reference's ChannelFirstAdaptor
computes, group_normalization.cu:93-106, instance_normalization.cu:81-94)."""
import numpy as np
import pytest
import torch

from _util import assert_close, dtype_name, load_package, rounded, to_dev, to_np
from oracle import norm_ref as R

pytestmark = pytest.mark.gpu
K = load_package()
DTYPES = [torch.float32, torch.float16]


def f32(a):
    return np.asarray(a, np.float32).astype(np.float64)


def to_cf(a):
    """[N, *spatial, C] -> [N, C, *spatial]"""
    return np.ascontiguousarray(np.moveaxis(a, -1, 1))


def to_cl(a):
    return np.ascontiguousarray(np.moveaxis(a, 1, -1))


def make_cl(n, sp, c, dtype, seed):
    rng = np.random.default_rng(seed)
    shape = (n,) + sp + (c,)
    x = rounded(rng.standard_normal(shape) * 1.5 + rng.uniform(-2, 2, (n,) + (1,) * len(sp) + (c,)),
                dtype)
    dy = rounded(rng.standard_normal(shape), dtype)
    g = f32(rng.uniform(0.5, 1.5, c))
    b = f32(rng.standard_normal(c) * 0.1)
    return x, dy, g, b


# (n, spatial, c, groups): packed loads with the fast apply (c/vec divides
# 256), packed loads with the generic apply (c = 24, 40), scalar loads (odd c),
# one row, one sample, several channel tiles (c = 2048), many row splits.
GN_CL_SHAPES = [(2, (8, 8), 8, 4), (3, (5,), 6, 2), (1, (2, 2), 4, 1), (2, (4,), 6, 6),
                (2, (7, 7), 32, 8), (2, (14, 14), 24, 4), (4, (16, 16), 64, 8),
                (2, (32, 32), 16, 2), (2, (64, 64), 256, 32), (1, (128, 128), 8, 1),
                (2, (512,), 12, 3), (2, (), 4, 2), (3, (64,), 10, 5), (1, (40, 40), 40, 2),
                (2, (3, 3), 2048, 32), (2, (4096,), 32, 4), (5, (33,), 7, 7), (1, (1,), 5, 1),
                # channel vectors that do not divide 256, rows wider than 256 vectors, 8-byte fp16 rows
                (2, (9, 9), 96, 4), (2, (5, 5), 4104, 8), (3, (11,), 100, 5), (2, (6, 6), 20, 2),
                # group cached in registers: 1 to 8 channel vectors per group, ragged last load,
                # groups that share cache lines (the XCD block map) and groups that do not
                (3, (33, 33), 64, 2), (2, (20, 20), 128, 2), (5, (17, 17), 16, 1), (3, (24, 24), 96, 12),
                (2, (56, 56), 64, 8), (9, (16, 16), 32, 4), (1, (90, 90), 8, 1),
                # half data, 8 channels per group, a block for every CU left: blocks that
                # take 2 or 4 neighbouring groups (ragged planes; the 1024 x 8 layout)
                (4, (32, 32), 1024, 128), (8, (33, 33), 1024, 128), (16, (64, 64), 256, 32),
                # groups that are no whole number of vectors, a block per range of
                # positions: 10, 20, 40, 80 and 6 channels per group, one to eleven
                # vectors per thread, ragged position counts, 64 groups
                (16, (16, 16), 320, 32), (8, (33, 31), 160, 16), (4, (40, 40), 640, 32),
                (8, (48, 48), 320, 32), (16, (32, 32), 1280, 32), (16, (16, 16), 2560, 32),
                (8, (32, 32), 192, 32), (4, (24, 24), 640, 64), (16, (61, 64), 320, 32)]


@pytest.mark.parametrize("n,sp,c,groups", GN_CL_SHAPES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_gn_channel_last(n, sp, c, groups, dtype):
    dn = dtype_name(dtype)
    x, dy, g, b = make_cl(n, sp, c, dtype, 11)
    xt, dyt = to_cf(x), to_cf(dy)
    y_r, m_r, v_r = R.gn_forward(xt, b, g, n, c, groups, 1e-5)
    dx_r, dg_r, db_r = R.gn_backward(xt, dyt, g, m_r, v_r, n, c, groups, 1e-5)
    xd, dyd, gd, bd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(b)
    y, m, v = K.gn_forward(xd, bd, gd, groups, 1e-5, channel_last=True)
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(y), to_cl(y_r.reshape(xt.shape)), dn, "y", "y")
    dx, dg, db = K.gn_backward(xd, dyd, gd, m, v, groups, 1e-5, channel_last=True)
    scale = 1.0 / np.sqrt(1e-5) if int(np.prod(sp)) * (c // groups) == 1 else None
    assert_close(to_np(dx), to_cl(dx_r.reshape(xt.shape)), dn, "grad", "dx", scale=scale)
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


IN_CL_SHAPES = [(2, (4, 4), 3), (3, (7,), 5), (1, (3, 2), 2), (4, (16, 16), 16), (2, (64, 64), 8),
                (2, (7, 7), 24), (1, (200, 200), 3), (2, (300, 300), 2), (3, (1,), 7),
                (2, (1000,), 64), (2, (5, 5), 1024), (16, (32, 32), 256),
                (2, (9, 9), 96), (2, (5, 5), 4104), (3, (11,), 100), (2, (300,), 1032),
                # instances cached in registers (256 positions and more)
                (3, (33, 33), 24), (2, (20, 20), 128), (5, (17, 17), 16), (2, (56, 56), 64),
                (1, (90, 90), 8), (9, (16, 16), 32),
                # half data, a block for every CU left: blocks of 2 or 4 channel vectors
                (4, (32, 32), 1024), (8, (33, 33), 1024), (16, (64, 32), 256)]


@pytest.mark.parametrize("n,sp,c", IN_CL_SHAPES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_in_channel_last(n, sp, c, dtype):
    dn = dtype_name(dtype)
    x, dy, g, b = make_cl(n, sp, c, dtype, 12)
    xt, dyt = to_cf(x), to_cf(dy)
    y_r, m_r, v_r = R.in_forward(xt, b, g, n, c, 1e-5)
    dx_r, dg_r, db_r = R.in_backward(xt, dyt, g, m_r, v_r, n, c, 1e-5)
    xd, dyd, gd, bd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(b)
    y, m, v = K.in_forward(xd, bd, gd, 1e-5, channel_last=True)
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(y), to_cl(y_r.reshape(xt.shape)), dn, "y", "y")
    dx, dg, db = K.in_backward(xd, dyd, gd, m, v, 1e-5, channel_last=True)
    scale = 1.0 / np.sqrt(1e-5) if int(np.prod(sp)) == 1 else None
    assert_close(to_np(dx), to_cl(dx_r.reshape(xt.shape)), dn, "grad", "dx", scale=scale)
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


@pytest.mark.parametrize("n,sp,c", [(3, (6, 6), 4), (2, (50, 50), 16)])
@pytest.mark.parametrize("bcg,bcb", [(False, False), (True, False), (False, True), (True, True)])
def test_in_channel_last_per_sample_parameters_and_flags(n, sp, c, bcg, bcb):
    rng = np.random.default_rng(7)
    shape = (n,) + sp + (c,)
    x = f32(rng.standard_normal(shape))
    dy = f32(rng.standard_normal(shape))
    g = f32(rng.uniform(0.5, 1.5, c if bcg else n * c))
    b = f32(rng.standard_normal(c if bcb else n * c))
    dm, dv = f32(rng.standard_normal(n * c)), f32(rng.standard_normal(n * c))
    g_full = np.tile(g, n) if bcg else g
    b_full = np.tile(b, n) if bcb else b
    xt, dyt = to_cf(x), to_cf(dy)
    y_r, m_r, v_r = R.in_forward(xt, b_full, g_full, n, c, 1e-5)
    dx_r, dg_r, db_r = R.in_backward(xt, dyt, g, m_r, v_r, n, c, 1e-5, dm, dv, bc_gamma=bcg,
                                     bc_beta=bcb)
    xd, dyd = to_dev(x), to_dev(dy)
    y, m, v = K.in_forward(xd, to_dev(b), to_dev(g), 1e-5, bc_gamma=bcg, bc_beta=bcb,
                           channel_last=True)
    assert_close(to_np(y), to_cl(y_r.reshape(xt.shape)), "f32", "y", "y")
    pre_g = rng.standard_normal(dg_r.size).astype(np.float32)
    dgd = to_dev(pre_g)
    dx, _, db = K.in_backward(xd, dyd, to_dev(g), m, v, 1e-5, bc_gamma=bcg, bc_beta=bcb,
                              dmean=to_dev(dm), dvar=to_dev(dv), dgamma=dgd,
                              accum=(False, True, False), channel_last=True)
    assert_close(to_np(dx), to_cl(dx_r.reshape(xt.shape)), "f32", "grad", "dx")
    assert_close(to_np(dgd), dg_r + pre_g, "f32", "pgrad", "dgamma accum")
    assert_close(to_np(db), db_r, "f32", "pgrad", "dbeta")


@pytest.mark.parametrize("n,sp,c,groups", [(4, (16, 16), 64, 8), (2, (7, 7), 24, 8), (8, (32, 32), 160, 16)])
def test_gn_channel_last_flags(n, sp, c, groups):
    """no_scale/no_bias, 3-output dmean/dvar, accumulation, propagate_down."""
    rng = np.random.default_rng(5)
    x, dy, g, b = make_cl(n, sp, c, torch.float32, 13)
    xt, dyt = to_cf(x), to_cf(dy)
    xd, dyd = to_dev(x), to_dev(dy)
    # no gamma, no beta
    y_r, m_r, v_r = R.gn_forward(xt, None, None, n, c, groups, 1e-5)
    y, m, v = K.gn_forward(xd, None, None, groups, 1e-5, channel_last=True)
    assert_close(to_np(y), to_cl(y_r.reshape(xt.shape)), "f32", "y", "y no params")
    dx_r, _, _ = R.gn_backward(xt, dyt, None, m_r, v_r, n, c, groups, 1e-5)
    dx, _, _ = K.gn_backward(xd, dyd, None, m, v, groups, 1e-5, need=(True, False, False),
                             channel_last=True)
    assert_close(to_np(dx), to_cl(dx_r.reshape(xt.shape)), "f32", "grad", "dx no params")
    # 3 outputs with accumulation
    dm, dv = f32(rng.standard_normal(n * groups)), f32(rng.standard_normal(n * groups))
    y_r, m_r, v_r = R.gn_forward(xt, b, g, n, c, groups, 1e-5)
    dx_r, dg_r, db_r = R.gn_backward(xt, dyt, g, m_r, v_r, n, c, groups, 1e-5, dm, dv)
    y, m, v = K.gn_forward(xd, to_dev(b), to_dev(g), groups, 1e-5, channel_last=True)
    pre_dx = rng.standard_normal(x.shape).astype(np.float32)
    pre_g = rng.standard_normal(c).astype(np.float32)
    pre_b = rng.standard_normal(c).astype(np.float32)
    dxd, dgd, dbd = to_dev(pre_dx), to_dev(pre_g), to_dev(pre_b)
    K.gn_backward(xd, dyd, to_dev(g), m, v, groups, 1e-5, dmean=to_dev(dm), dvar=to_dev(dv), dx=dxd,
                  dgamma=dgd, dbeta=dbd, accum=(True, True, True), channel_last=True)
    assert_close(to_np(dxd), to_cl(dx_r.reshape(xt.shape)) + pre_dx, "f32", "grad", "dx accum")
    assert_close(to_np(dgd), dg_r + pre_g, "f32", "pgrad", "dgamma accum")
    assert_close(to_np(dbd), db_r + pre_b, "f32", "pgrad", "dbeta accum")
    _, dg, db = K.gn_backward(xd, dyd, to_dev(g), m, v, groups, 1e-5, dmean=to_dev(dm),
                              dvar=to_dev(dv), need=(False, True, True), channel_last=True)
    assert_close(to_np(dg), dg_r, "f32", "pgrad", "dgamma only")
    assert_close(to_np(db), db_r, "f32", "pgrad", "dbeta only")


def test_channel_last_matches_channel_first_entry_points():
    """Same tensor through both layouts: statistics agree to rounding, outputs
    agree after the transpose, and a repeated call is bit-identical."""
    torch.manual_seed(2)
    x = torch.randn(4, 32, 24, 24, device="cuda")
    dy = torch.randn_like(x)
    g = torch.rand(32, device="cuda") + 0.5
    b = torch.randn(32, device="cuda")
    xl = x.permute(0, 2, 3, 1).contiguous()
    dyl = dy.permute(0, 2, 3, 1).contiguous()
    y1, m1, v1 = K.gn_forward(x, b, g, 4, 1e-5)
    y2, m2, v2 = K.gn_forward(xl, b, g, 4, 1e-5, channel_last=True)
    torch.testing.assert_close(m1, m2, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(v1, v2, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(y1, y2.permute(0, 3, 1, 2), rtol=1e-5, atol=1e-5)
    dx1, dg1, db1 = K.gn_backward(x, dy, g, m1, v1, 4, 1e-5)
    dx2, dg2, db2 = K.gn_backward(xl, dyl, g, m2, v2, 4, 1e-5, channel_last=True)
    torch.testing.assert_close(dx1, dx2.permute(0, 3, 1, 2), rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(dg1, dg2, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(db1, db2, rtol=1e-4, atol=1e-4)
    y3, m3, v3 = K.gn_forward(xl, b, g, 4, 1e-5, channel_last=True)
    dx3, dg3, db3 = K.gn_backward(xl, dyl, g, m3, v3, 4, 1e-5, channel_last=True)
    for a, c in ((y2, y3), (m2, m3), (v2, v3), (dx2, dx3), (dg2, dg3), (db2, db3)):
        assert torch.equal(a, c)


def test_channel_last_misaligned_pointer():
    """Pointers off the 16-byte grid take the scalar-load kernels."""
    n, sp, c, groups = 2, (9, 9), 16, 4
    x, dy, g, b = make_cl(n, sp, c, torch.float16, 21)
    xt, dyt = to_cf(x), to_cf(dy)
    y_r, m_r, v_r = R.gn_forward(xt, b, g, n, c, groups, 1e-5)
    dx_r, dg_r, db_r = R.gn_backward(xt, dyt, g, m_r, v_r, n, c, groups, 1e-5)
    numel = x.size
    bx = torch.empty(numel + 8, dtype=torch.float16, device="cuda")
    bdy = torch.empty(numel + 8, dtype=torch.float16, device="cuda")
    xd = bx[1:1 + numel].view(x.shape)
    dyd = bdy[1:1 + numel].view(x.shape)
    xd.copy_(to_dev(x, torch.float16))
    dyd.copy_(to_dev(dy, torch.float16))
    assert xd.data_ptr() % 16 != 0 and xd.is_contiguous()
    y, m, v = K.gn_forward(xd, to_dev(b), to_dev(g), groups, 1e-5, channel_last=True)
    assert_close(to_np(y), to_cl(y_r.reshape(xt.shape)), "f16", "y", "y")
    dx, dg, db = K.gn_backward(xd, dyd, to_dev(g), m, v, groups, 1e-5, channel_last=True)
    assert_close(to_np(dx), to_cl(dx_r.reshape(xt.shape)), "f16", "grad", "dx")
    assert_close(to_np(dg), dg_r, "f16", "pgrad", "dgamma")
    assert_close(to_np(db), db_r, "f16", "pgrad", "dbeta")


def test_c4_channel_last_full_size():
    """Benchmark configuration 4 stored channel-last: x[16,64,64,256] fp16, GN with 32
    groups and IN, seed 3."""
    rng = np.random.default_rng(3)
    n, c, sp = 16, 256, (64, 64)
    x = (rng.standard_normal((n,) + sp + (c,), dtype=np.float32) * 1.5).astype(np.float16)
    dy = rng.standard_normal((n,) + sp + (c,), dtype=np.float32).astype(np.float16)
    g = rng.uniform(0.5, 1.5, c).astype(np.float32)
    b = (rng.standard_normal(c) * 0.1).astype(np.float32)
    xd, dyd = torch.from_numpy(x).cuda(), torch.from_numpy(dy).cuda()
    gd, bd = to_dev(g), to_dev(b)
    xt, dyt = to_cf(x), to_cf(dy)
    y, m, v = K.gn_forward(xd, bd, gd, 32, 1e-5, channel_last=True)
    dx, dg, db = K.gn_backward(xd, dyd, gd, m, v, 32, 1e-5, channel_last=True)
    y_r, m_r, v_r = R.gn_forward(xt, b, g, n, c, 32, 1e-5)
    dx_r, dg_r, db_r = R.gn_backward(xt, dyt, g, m_r, v_r, n, c, 32, 1e-5)
    assert_close(to_np(m), m_r, "f16", "stat", "gn mean")
    assert_close(to_np(v), v_r, "f16", "stat", "gn var")
    assert_close(to_np(y), to_cl(y_r.reshape(xt.shape)), "f16", "y", "gn y")
    assert_close(to_np(dx), to_cl(dx_r.reshape(xt.shape)), "f16", "grad", "gn dx")
    assert_close(to_np(dg), dg_r, "f16", "pgrad", "gn dgamma")
    assert_close(to_np(db), db_r, "f16", "pgrad", "gn dbeta")
    y, m, v = K.in_forward(xd, bd, gd, 1e-5, channel_last=True)
    dx, dg, db = K.in_backward(xd, dyd, gd, m, v, 1e-5, channel_last=True)
    y_r, m_r, v_r = R.in_forward(xt, b, g, n, c, 1e-5)
    dx_r, dg_r, db_r = R.in_backward(xt, dyt, g, m_r, v_r, n, c, 1e-5)
    assert_close(to_np(m), m_r, "f16", "stat", "in mean")
    assert_close(to_np(v), v_r, "f16", "stat", "in var")
    assert_close(to_np(y), to_cl(y_r.reshape(xt.shape)), "f16", "y", "in y")
    assert_close(to_np(dx), to_cl(dx_r.reshape(xt.shape)), "f16", "grad", "in dx")
    assert_close(to_np(dg), dg_r, "f16", "pgrad", "in dgamma")
    assert_close(to_np(db), db_r, "f16", "pgrad", "in dbeta")


def test_channel_last_argument_errors():
    L = K.lib()
    s = torch.cuda.current_stream().cuda_stream
    x = torch.randn(2, 16, 8, device="cuda")
    y = torch.empty_like(x)
    m = torch.empty(16, device="cuda")
    ws = torch.empty(L.nblahip_gn_cl_workspace_bytes(2, 16, 8, 4, 0), dtype=torch.uint8,
                     device="cuda")
    assert ws.numel() > 0
    assert L.nblahip_gn_cl_fwd(x.data_ptr(), None, None, y.data_ptr(), m.data_ptr(), m.data_ptr(),
                               2, 16, 8, 3, 1e-5, 0, ws.data_ptr(), ws.numel(), s) == -1  # 8 % 3
    assert L.nblahip_gn_cl_fwd(x.data_ptr(), None, None, y.data_ptr(), m.data_ptr(), m.data_ptr(),
                               2, 16, 8, 4, 1e-5, 0, None, 0, s) == -2          # no workspace
    assert L.nblahip_gn_cl_fwd(x.data_ptr(), None, None, y.data_ptr(), m.data_ptr(), m.data_ptr(),
                               2, 16, 8, 4, 1e-5, 0, ws.data_ptr(), 16, s) == -2  # too small
    assert L.nblahip_gn_cl_fwd(x.data_ptr(), None, None, y.data_ptr(), m.data_ptr(), m.data_ptr(),
                               0, 16, 8, 4, 1e-5, 0, None, 0, s) == 0           # empty: no-op
    # (a batch beyond 65535 runs in ranges of samples; it needs its own workspace)
    assert L.nblahip_in_cl_workspace_bytes(70000, 1, 8, 0) > ws.numel()
    # (y = x: with these sizes the two small buffers would overlap in part)
    assert L.nblahip_in_cl_fwd(x.data_ptr(), None, None, x.data_ptr(), m.data_ptr(), m.data_ptr(),
                               70000, 1, 8, 1, 1, 1e-5, 0, ws.data_ptr(), ws.numel(),
                               s) == -2
    assert L.nblahip_in_cl_fwd(x.data_ptr(), None, None, x.data_ptr(), m.data_ptr(), m.data_ptr(),
                               2, 1 << 16, 1 << 15, 1, 1, 1e-5, 0, ws.data_ptr(), ws.numel(),
                               s) == -3                                         # 2^31 elements per sample
    assert L.nblahip_in_cl_bwd(x.data_ptr(), None, None, m.data_ptr(), m.data_ptr(), None, None,
                               y.data_ptr(), None, None, 0, 0, 0, 2, 16, 8, 1, 1, 1e-5, 0,
                               ws.data_ptr(), ws.numel(), s) == -1              # dy missing
