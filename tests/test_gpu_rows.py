"""LayerNormalization / GroupNormalization / InstanceNormalization parity on
the GPU: HIP path through the C-ABI against the float64 oracle."""
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


# ------------------------------------------------------------------ LN
# (outer, R): below one wave, odd (scalar loads), one wave per row, one block
# per row (256 / 1024 threads), longer than the register-cached limit
# (streaming kernels), single row, R == 1.
LN_SHAPES = [(5, 1), (7, 3), (16, 17), (33, 64), (9, 1000), (64, 1024), (130, 768), (12, 4096),
             (5, 8192), (3, 16384), (6, 32768), (2, 70000), (3, 40004), (1, 2048), (300, 256),
             (2, 131072),
             # half rows of 4k (not 8k) elements: 8-byte loads
             (40, 1004), (9, 20), (70, 516), (4, 8196), (3, 2052),
             # several rows per wave (4 to 32 lanes each), ragged row counts
             (1000, 32), (513, 128), (100, 48), (77, 200), (2049, 64), (31, 8), (129, 24), (65, 392)]


def make_ln(outer, Rr, dtype, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((outer, Rr)) + rng.uniform(-3, 3, (outer, 1))
    dy = rng.standard_normal((outer, Rr))
    g = f32(rng.standard_normal(Rr) * 0.1 + 1)
    b = f32(rng.standard_normal(Rr) * 0.1)
    return rounded(x, dtype), rounded(dy, dtype), g, b


@pytest.mark.parametrize("outer,Rr", LN_SHAPES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_ln_forward_backward(outer, Rr, dtype):
    dn = dtype_name(dtype)
    x, dy, g, b = make_ln(outer, Rr, dtype, 2)
    y_r, m_r, v_r = R.ln_forward(x, b, g, outer, 1e-5)
    dx_r, dg_r, db_r = R.ln_backward(x, dy, g, m_r, v_r, outer, 1e-5)
    xd, dyd, gd, bd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(b)
    y, m, v = K.ln_forward(xd, bd, gd, outer, 1e-5)
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(y), y_r, dn, "y", "y")
    dx, dg, db = K.ln_backward(xd, dyd, gd, m, v, outer, 1e-5)
    # One element per row: var == 0 and dx is the exact cancellation of two
    # terms of size |dy*gamma|/sqrt(eps); the floor follows that size.
    scale = 1.0 / np.sqrt(1e-5) if Rr == 1 else None
    assert_close(to_np(dx), dx_r, dn, "grad", "dx", scale=scale)
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


@pytest.mark.parametrize("outer,Rr", [(33, 64), (9, 1000), (12, 4096), (2, 70000)])
def test_ln_flags(outer, Rr):
    """no_scale/no_bias, 3-output dmean/dvar, accumulation, propagate_down."""
    dtype = torch.float32
    x, dy, g, b = make_ln(outer, Rr, dtype, 3)
    rng = np.random.default_rng(4)
    dm, dv = f32(rng.standard_normal(outer)), f32(rng.standard_normal(outer))
    xd, dyd = to_dev(x), to_dev(dy)
    y_r, m_r, v_r = R.ln_forward(x, None, None, outer, 1e-5)
    y, m, v = K.ln_forward(xd, None, None, outer, 1e-5)
    assert_close(to_np(y), y_r, "f32", "y", "y no affine")
    dx_r, dg_r, db_r = R.ln_backward(x, dy, None, m_r, v_r, outer, 1e-5, dm, dv)
    dx, dg, db = K.ln_backward(xd, dyd, None, m, v, outer, 1e-5, dmean=to_dev(dm), dvar=to_dev(dv))
    assert_close(to_np(dx), dx_r, "f32", "grad", "dx 3-output")
    assert_close(to_np(dg), dg_r, "f32", "pgrad", "dgamma")
    assert_close(to_np(db), db_r, "f32", "pgrad", "dbeta")

    dx_r, dg_r, db_r = R.ln_backward(x, dy, g, m_r, v_r, outer, 1e-5)
    pre_dx = rng.standard_normal((outer, Rr)).astype(np.float32)
    pre_g = rng.standard_normal(Rr).astype(np.float32)
    pre_b = rng.standard_normal(Rr).astype(np.float32)
    dxd, dgd, dbd = to_dev(pre_dx), to_dev(pre_g), to_dev(pre_b)
    K.ln_backward(xd, dyd, to_dev(g), m, v, outer, 1e-5, dx=dxd, dgamma=dgd, dbeta=dbd,
                  accum=(True, True, True))
    assert_close(to_np(dxd), dx_r + pre_dx, "f32", "grad", "dx accum")
    assert_close(to_np(dgd), dg_r + pre_g, "f32", "pgrad", "dgamma accum")
    assert_close(to_np(dbd), db_r + pre_b, "f32", "pgrad", "dbeta accum")

    _, dg, db = K.ln_backward(xd, dyd, to_dev(g), m, v, outer, 1e-5, need=(False, True, True))
    assert_close(to_np(dg), dg_r, "f32", "pgrad", "dgamma only")
    dx, _, _ = K.ln_backward(xd, dyd, to_dev(g), m, v, outer, 1e-5, need=(True, False, False))
    assert_close(to_np(dx), dx_r, "f32", "grad", "dx only")


def test_ln_invariants_and_determinism():
    torch.manual_seed(0)
    x = torch.randn(512, 1024, device="cuda")
    dy = torch.randn(512, 1024, device="cuda")
    y, m, v = K.ln_forward(x, None, None, 512, 1e-5)
    # normalised rows: mean 0, var = var/(var+eps)
    assert y.mean(dim=1).abs().max().item() < 1e-5
    dx, dg, db = K.ln_backward(x, dy, None, m, v, 512, 1e-5)
    assert dx.sum(dim=1).abs().max().item() < 1e-3
    dx2, dg2, db2 = K.ln_backward(x, dy, None, m, v, 512, 1e-5)
    assert torch.equal(dx, dx2) and torch.equal(dg, dg2) and torch.equal(db, db2)
    # constant rows give y == beta exactly
    xc = torch.full((8, 256), 3.25, device="cuda")
    b = torch.linspace(-1, 1, 256, device="cuda")
    yc, _, vc = K.ln_forward(xc, b, torch.ones(256, device="cuda"), 8, 1e-5)
    assert torch.equal(vc, torch.zeros_like(vc))
    assert torch.equal(yc, b.expand(8, 256).contiguous())


def test_ln_misaligned_pointer():
    rng = np.random.default_rng(6)
    outer, Rr = 8, 1024
    flat = rng.standard_normal(outer * Rr + 1).astype(np.float32)
    xd = to_dev(flat)[1:].view(outer, Rr)
    assert xd.data_ptr() % 16 != 0
    x = flat[1:].reshape(outer, Rr).astype(np.float64)
    y_r, m_r, v_r = R.ln_forward(x, None, None, outer, 1e-5)
    y, m, v = K.ln_forward(xd, None, None, outer, 1e-5)
    assert_close(to_np(y), y_r, "f32", "y", "y")
    assert_close(to_np(v), v_r, "f32", "stat", "var")


@pytest.mark.parametrize("dtype", DTYPES)
def test_ln_c3_full_size(dtype):
    """Benchmark configuration 3: x[32,512,1024] ~ N(0,1) + per-row offset U(-3,3),
    gamma ~ N(1,0.1), beta ~ N(0,0.1), seed 2, fp32 and fp16."""
    dn = dtype_name(dtype)
    rng = np.random.default_rng(2)
    outer, Rr = 32 * 512, 1024
    x = rng.standard_normal((outer, Rr), dtype=np.float32) + \
        rng.uniform(-3, 3, (outer, 1)).astype(np.float32)
    dy = rng.standard_normal((outer, Rr), dtype=np.float32)
    g = (rng.standard_normal(Rr) * 0.1 + 1).astype(np.float32)
    b = (rng.standard_normal(Rr) * 0.1).astype(np.float32)
    x, dy = rounded(x, dtype), rounded(dy, dtype)
    y_r, m_r, v_r = R.ln_forward(x, b, g, outer, 1e-5)
    dx_r, dg_r, db_r = R.ln_backward(x, dy, g, m_r, v_r, outer, 1e-5)
    xd, dyd, gd, bd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(b)
    y, m, v = K.ln_forward(xd, bd, gd, outer, 1e-5)
    dx, dg, db = K.ln_backward(xd, dyd, gd, m, v, outer, 1e-5)
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(y), y_r, dn, "y", "y")
    assert_close(to_np(dx), dx_r, dn, "grad", "dx")
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


# ------------------------------------------------------------------ GN
# (n, c, spatial-shape, groups): register-cached with wave-uniform channels,
# spatial that is not (49, 196), one channel per group, one group, tiny, big
# groups that stream.
GN_SHAPES = [(2, 8, (8, 8), 4), (3, 6, (5,), 2), (1, 4, (2, 2), 1), (2, 6, (4,), 6),
             (2, 32, (7, 7), 8), (2, 32, (14, 14), 4), (4, 64, (16, 16), 8), (2, 16, (32, 32), 2),
             (2, 256, (64, 64), 32), (1, 8, (128, 128), 1), (2, 12, (512,), 3), (2, 4, (), 2),
             (3, 10, (64,), 5), (1, 64, (40, 40), 2),
             # thread maps of the backward: several channels per wave, several waves per
             # channel, wave sets that do not divide the block, planes that end inside a load
             (2, 64, (56, 56), 8), (2, 64, (28, 28), 4), (2, 6, (8, 8), 2), (2, 4, (64, 64), 4),
             (1, 10, (48, 48), 2), (2, 64, (14, 14), 2), (2, 128, (7, 7), 2), (1, 80, (8, 8), 2),
             (3, 24, (24, 24), 3), (2, 14, (72,), 2),
             # float groups of 64-128 KB: 1024 threads x 8 loads, dy parked in LDS (fixed map)
             (2, 16, (64, 64), 2),
             # planes of 8, 16 and 32 vectors with the group held on one CU in the backward:
             # 2, 4 or 8 channels side by side in a wave's load
             (4, 2560, (16, 16), 32), (2, 4096, (8, 16), 32), (4, 2048, (16, 8), 16),
             (4, 2048, (8, 8), 16),
             # one group of 2M elements per sample: split streaming reductions
             (2, 32, (256, 256), 1), (1, 6, (333, 333), 2),
             # planes that are no whole number of vectors, taken with the tensor's aligned
             # vectors (a channel boundary inside a vector); short planes: the forward only
             (2, 16, (63, 63), 4), (4, 32, (33, 33), 8), (2, 8, (17, 17), 2), (3, 6, (5, 7), 3),
             (2, 256, (63, 63), 32), (1, 24, (65, 65), 3), (3, 9, (31, 33), 3), (2, 12, (127, 9), 2),
             # ... several planes per wave (8, 16, 32 threads per plane), up to 64 channels per group
             (4, 1280, (15, 15), 32), (8, 512, (7, 7), 32), (4, 60, (9, 9), 6), (3, 48, (5, 5), 3),
             (2, 128, (11, 13), 2), (2, 40, (17, 19), 1), (2, 8, (127, 127), 2)]


def make_nc(n, c, sp, dtype, seed):
    rng = np.random.default_rng(seed)
    shape = (n, c) + sp
    x = rounded(rng.standard_normal(shape) * 1.5, dtype)
    dy = rounded(rng.standard_normal(shape), dtype)
    g = f32(rng.uniform(0.5, 1.5, c))
    b = f32(rng.standard_normal(c) * 0.1)
    return x, dy, g, b


@pytest.mark.parametrize("n,c,sp,groups", GN_SHAPES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_gn_forward_backward(n, c, sp, groups, dtype):
    dn = dtype_name(dtype)
    x, dy, g, b = make_nc(n, c, sp, dtype, 3)
    y_r, m_r, v_r = R.gn_forward(x, b, g, n, c, groups, 1e-5)
    dx_r, dg_r, db_r = R.gn_backward(x, dy, g, m_r, v_r, n, c, groups, 1e-5)
    xd, dyd, gd, bd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(b)
    y, m, v = K.gn_forward(xd, bd, gd, groups, 1e-5)
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(y), y_r, dn, "y", "y")
    dx, dg, db = K.gn_backward(xd, dyd, gd, m, v, groups, 1e-5)
    assert_close(to_np(dx), dx_r, dn, "grad", "dx")
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


@pytest.mark.parametrize("n,c,sp,groups", [(4, 64, (16, 16), 8), (2, 32, (7, 7), 8),
                                           (2, 160, (64, 64), 16),
                                           # the group held on one CU in the backward
                                           (4, 320, (64, 64), 32),
                                           # planes that are no whole number of vectors
                                           (2, 16, (33, 31), 4)])
def test_gn_flags(n, c, sp, groups):
    dtype = torch.float32
    x, dy, g, b = make_nc(n, c, sp, dtype, 5)
    rng = np.random.default_rng(6)
    rows = n * groups
    dm, dv = f32(rng.standard_normal(rows)), f32(rng.standard_normal(rows))
    xd, dyd = to_dev(x), to_dev(dy)
    y_r, m_r, v_r = R.gn_forward(x, None, None, n, c, groups, 1e-5)
    y, m, v = K.gn_forward(xd, None, None, groups, 1e-5)
    assert_close(to_np(y), y_r, "f32", "y", "y no affine")
    dx_r, dg_r, db_r = R.gn_backward(x, dy, g, m_r, v_r, n, c, groups, 1e-5, dm, dv)
    pre_dx = rng.standard_normal(x.shape).astype(np.float32)
    pre_g = rng.standard_normal(c).astype(np.float32)
    pre_b = rng.standard_normal(c).astype(np.float32)
    dxd, dgd, dbd = to_dev(pre_dx), to_dev(pre_g), to_dev(pre_b)
    K.gn_backward(xd, dyd, to_dev(g), m, v, groups, 1e-5, dmean=to_dev(dm), dvar=to_dev(dv), dx=dxd,
                  dgamma=dgd, dbeta=dbd, accum=(True, True, True))
    assert_close(to_np(dxd), dx_r + pre_dx, "f32", "grad", "dx accum 3-output")
    assert_close(to_np(dgd), dg_r + pre_g, "f32", "pgrad", "dgamma accum")
    assert_close(to_np(dbd), db_r + pre_b, "f32", "pgrad", "dbeta accum")
    _, dg, db = K.gn_backward(xd, dyd, to_dev(g), m, v, groups, 1e-5, dmean=to_dev(dm),
                              dvar=to_dev(dv), need=(False, True, True))
    assert_close(to_np(dg), dg_r, "f32", "pgrad", "dgamma only")
    assert_close(to_np(db), db_r, "f32", "pgrad", "dbeta only")


# ------------------------------------------------------------------ IN
IN_SHAPES = [(2, 3, (4, 4)), (3, 5, (7,)), (1, 2, (3, 2)), (4, 16, (16, 16)), (2, 8, (64, 64)),
             (2, 4, (7, 7)), (1, 3, (200, 200)), (2, 2, (300, 300)), (3, 7, (1,)), (2, 3, (1000,)),
             (4, 8, (14, 14)), (2, 3, (6, 6)), (2, 300, (14, 14)), (3, 2, (90, 90)),
             (8, 64, (8, 8)), (5, 33, (7, 7)), (3, 300, (4, 4)), (2, 129, (3, 5)), (7, 11, (6,)),
             # a few very long rows: split streaming reductions
             (2, 4, (64, 64, 64)), (1, 2, (999, 1001)),
             # planes that are no whole number of vectors, taken with the tensor's aligned
             # vectors: one wave to 1024 threads per row, a tensor that ends inside a vector
             (3, 5, (7, 7)), (2, 3, (5, 5)), (6, 10, (9, 7)), (16, 64, (63, 63)), (4, 8, (65, 65)),
             (2, 4, (129, 129)), (1, 3, (255, 255)), (3, 2, (181, 90))]


@pytest.mark.parametrize("n,c,sp", IN_SHAPES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_in_forward_backward(n, c, sp, dtype):
    dn = dtype_name(dtype)
    x, dy, g, b = make_nc(n, c, sp, dtype, 3)
    y_r, m_r, v_r = R.in_forward(x, b, g, n, c, 1e-5)
    dx_r, dg_r, db_r = R.in_backward(x, dy, g, m_r, v_r, n, c, 1e-5)
    xd, dyd, gd, bd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(b)
    y, m, v = K.in_forward(xd, bd, gd, 1e-5)
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(y), y_r, dn, "y", "y")
    dx, dg, db = K.in_backward(xd, dyd, gd, m, v, 1e-5)
    # One element per plane: var == 0 and dx is the exact cancellation of two
    # terms of size |dy*gamma|/sqrt(eps); the floor follows that size.
    scale = 1.0 / np.sqrt(1e-5) if int(np.prod(sp)) == 1 else None
    assert_close(to_np(dx), dx_r, dn, "grad", "dx", scale=scale)
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


@pytest.mark.parametrize("n,c,sp", [(3, 4, (6, 6)), (2, 3, (300, 300)), (2, 32, (190, 190)),
                                    (2, 6, (33, 31))])
@pytest.mark.parametrize("bcg,bcb", [(False, False), (True, False), (False, True)])
def test_in_per_sample_parameters_and_flags(n, c, sp, bcg, bcb):
    """gamma/beta of batch*channels elements (no broadcast over the batch),
    mixed broadcast, 3-output dmean/dvar and accumulation."""
    dtype = torch.float32
    rng = np.random.default_rng(7)
    shape = (n, c) + sp
    x = f32(rng.standard_normal(shape))
    dy = f32(rng.standard_normal(shape))
    g = f32(rng.uniform(0.5, 1.5, c if bcg else n * c))
    b = f32(rng.standard_normal(c if bcb else n * c))
    dm, dv = f32(rng.standard_normal(n * c)), f32(rng.standard_normal(n * c))
    g_full = np.tile(g, n) if bcg else g
    b_full = np.tile(b, n) if bcb else b
    y_r, m_r, v_r = R.in_forward(x, b_full, g_full, n, c, 1e-5)
    dx_r, dg_r, db_r = R.in_backward(x, dy, g, m_r, v_r, n, c, 1e-5, dm, dv, bc_gamma=bcg,
                                     bc_beta=bcb)
    xd, dyd = to_dev(x), to_dev(dy)
    y, m, v = K.in_forward(xd, to_dev(b), to_dev(g), 1e-5, bc_gamma=bcg, bc_beta=bcb)
    assert_close(to_np(y), y_r, "f32", "y", "y")
    pre_g = rng.standard_normal(dg_r.size).astype(np.float32)
    dgd = to_dev(pre_g)
    dx, _, db = K.in_backward(xd, dyd, to_dev(g), m, v, 1e-5, bc_gamma=bcg, bc_beta=bcb,
                              dmean=to_dev(dm), dvar=to_dev(dv), dgamma=dgd,
                              accum=(False, True, False))
    assert_close(to_np(dx), dx_r, "f32", "grad", "dx")
    assert_close(to_np(dgd), dg_r + pre_g, "f32", "pgrad", "dgamma accum")
    assert_close(to_np(db), db_r, "f32", "pgrad", "dbeta")


def test_c4_gn_and_in_full_size():
    """Benchmark configuration 4: x[16,256,64,64] ~ N(0,1.5) fp16, GN with 32 groups and
    IN on the same tensor, seed 3."""
    rng = np.random.default_rng(3)
    n, c, sp = 16, 256, (64, 64)
    x = (rng.standard_normal((n, c) + sp, dtype=np.float32) * 1.5).astype(np.float16)
    dy = rng.standard_normal((n, c) + sp, dtype=np.float32).astype(np.float16)
    g = rng.uniform(0.5, 1.5, c).astype(np.float32)
    b = (rng.standard_normal(c) * 0.1).astype(np.float32)
    xd, dyd = torch.from_numpy(x).cuda(), torch.from_numpy(dy).cuda()
    gd, bd = to_dev(g), to_dev(b)
    # GroupNormalization
    y, m, v = K.gn_forward(xd, bd, gd, 32, 1e-5)
    dx, dg, db = K.gn_backward(xd, dyd, gd, m, v, 32, 1e-5)
    y_r, m_r, v_r = R.gn_forward(x, b, g, n, c, 32, 1e-5)
    dx_r, dg_r, db_r = R.gn_backward(x, dy, g, m_r, v_r, n, c, 32, 1e-5)
    assert_close(to_np(m), m_r, "f16", "stat", "gn mean")
    assert_close(to_np(v), v_r, "f16", "stat", "gn var")
    assert_close(to_np(y), y_r, "f16", "y", "gn y")
    assert_close(to_np(dx), dx_r, "f16", "grad", "gn dx")
    assert_close(to_np(dg), dg_r, "f16", "pgrad", "gn dgamma")
    assert_close(to_np(db), db_r, "f16", "pgrad", "gn dbeta")
    # InstanceNormalization
    y, m, v = K.in_forward(xd, bd, gd, 1e-5)
    dx, dg, db = K.in_backward(xd, dyd, gd, m, v, 1e-5)
    y_r, m_r, v_r = R.in_forward(x, b, g, n, c, 1e-5)
    dx_r, dg_r, db_r = R.in_backward(x, dy, g, m_r, v_r, n, c, 1e-5)
    assert_close(to_np(m), m_r, "f16", "stat", "in mean")
    assert_close(to_np(v), v_r, "f16", "stat", "in var")
    assert_close(to_np(y), y_r, "f16", "y", "in y")
    assert_close(to_np(dx), dx_r, "f16", "grad", "in dx")
    assert_close(to_np(dg), dg_r, "f16", "pgrad", "in dgamma")
    assert_close(to_np(db), db_r, "f16", "pgrad", "in dbeta")


def test_gn_with_one_channel_per_group_equals_in():
    torch.manual_seed(1)
    x = torch.randn(4, 16, 16, 16, device="cuda")
    g = torch.rand(16, device="cuda") + 0.5
    b = torch.randn(16, device="cuda")
    y1, m1, v1 = K.gn_forward(x, b, g, 16, 1e-5)
    y2, m2, v2 = K.in_forward(x, b, g, 1e-5)
    assert torch.equal(y1, y2) and torch.equal(m1, m2) and torch.equal(v1, v2)


def test_row_argument_errors():
    L = K.lib()
    s = torch.cuda.current_stream().cuda_stream
    x = torch.randn(8, 64, device="cuda")
    y = torch.empty_like(x)
    m = torch.empty(8, device="cuda")
    assert L.nblahip_ln_fwd(x.data_ptr(), None, None, y.data_ptr(), m.data_ptr(), None, 8, 64,
                            1e-5, 0, s) == -1                      # var missing
    assert L.nblahip_gn_fwd(x.data_ptr(), None, None, y.data_ptr(), m.data_ptr(), m.data_ptr(), 1,
                            8, 64, 3, 1e-5, 0, s) == -1            # 8 channels, 3 groups
    assert L.nblahip_ln_fwd(x.data_ptr(), None, None, y.data_ptr(), m.data_ptr(), m.data_ptr(), 0,
                            64, 1e-5, 0, s) == 0                   # empty: no-op
    assert L.nblahip_ln_bwd(x.data_ptr(), x.data_ptr(), None, m.data_ptr(), m.data_ptr(), None,
                            None, y.data_ptr(), None, None, 0, 0, 0, 8, 64, 1e-5, 0, None, 0,
                            s) == -2                               # workspace missing
    assert L.nblahip_ln_fwd(x.data_ptr(), None, None, y.data_ptr(), m.data_ptr(), m.data_ptr(),
                            2, 1 << 31, 1e-5, 0, s) == -3          # >= 2^31 elements per row


@pytest.mark.parametrize("outer,Rr", [(64, 1024), (300, 48), (2, 131072), (3, 40004)])
def test_ln_forward_in_place(outer, Rr):
    """y == x: register-cached, several rows per wave, and the streaming path
    (which must then not keep its partial statistics in y)."""
    x, _, g, b = make_ln(outer, Rr, torch.float32, 31)
    y_r, m_r, v_r = R.ln_forward(x, b, g, outer, 1e-5)
    xd, gd, bd = to_dev(x), to_dev(g), to_dev(b)
    mean = torch.empty(outer, device="cuda")
    var = torch.empty(outer, device="cuda")
    L = K.lib()
    K.check(L.nblahip_ln_fwd(xd.data_ptr(), gd.data_ptr(), bd.data_ptr(), xd.data_ptr(),
                             mean.data_ptr(), var.data_ptr(), outer, Rr, 1e-5, 0,
                             torch.cuda.current_stream().cuda_stream))
    assert_close(to_np(xd), y_r, "f32", "y", "y in place")
    assert_close(to_np(mean), m_r, "f32", "stat", "mean")
    assert_close(to_np(var), v_r, "f32", "stat", "var")


# Many rows of a few KB: a few blocks per CU walk the rows and ask for their next
# row ahead.  Two and three blocks per CU, a block and a wave per row, 1 to 4
# vectors per thread, a last round that not every block takes part in.
@pytest.mark.parametrize("outer,Rr,dtype", [(1501, 4096, torch.float16), (2100, 3072, torch.float16),
                                            (1203, 6144, torch.float16), (1101, 8192, torch.float16),
                                            (7003, 768, torch.float16), (9001, 1024, torch.float16),
                                            (1333, 4096, torch.float32), (1100, 3072, torch.float32),
                                            (1250, 2560, torch.float32), (1037, 16384, torch.float16)])
def test_ln_forward_rows_ahead(outer, Rr, dtype):
    """Against the oracle; bit for bit what the block-per-row launch gives
    (same arithmetic per row); in place as well."""
    dn = dtype_name(dtype)
    x, _, g, b = make_ln(outer, Rr, dtype, 41)
    y_r, m_r, v_r = R.ln_forward(x, b, g, outer, 1e-5)
    xd, gd, bd = to_dev(x, dtype), to_dev(g), to_dev(b)
    try:
        K.tune_reset()
        y, m, v = K.ln_forward(xd, bd, gd, outer, 1e-5)
        K.tune_set("LN_FWD_AHEAD", 0)
        y0, m0, v0 = K.ln_forward(xd, bd, gd, outer, 1e-5)
        K.tune_reset()
        L = K.lib()
        xin = xd.clone()
        mi, vi = torch.empty(outer, device="cuda"), torch.empty(outer, device="cuda")
        K.check(L.nblahip_ln_fwd(xin.data_ptr(), gd.data_ptr(), bd.data_ptr(), xin.data_ptr(),
                                 mi.data_ptr(), vi.data_ptr(), outer, Rr, 1e-5, K._dtype_code(xin),
                                 torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
    finally:
        K.tune_reset()
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(y), y_r, dn, "y", "y")
    assert torch.equal(y, y0) and torch.equal(m, m0) and torch.equal(v, v0)
    assert torch.equal(xin, y) and torch.equal(mi, m) and torch.equal(vi, v)


# ... and the backward with two or three vectors per thread: a wave and a block
# per row, a last round that not every block takes part in.
@pytest.mark.parametrize("outer,Rr,dtype", [(9001, 1024, torch.float16), (5003, 768, torch.float32),
                                            (1301, 8192, torch.float16), (1203, 5120, torch.float16),
                                            (1100, 5120, torch.float32), (1501, 4096, torch.float32),
                                            (2100, 6144, torch.float16)])
def test_ln_backward_rows_ahead(outer, Rr, dtype):
    """Against the oracle, with the statistics' gradients; close to what the
    kernel without the rows ahead gives (that one keeps dy*gamma of a short row
    in registers, this one multiplies gamma*istd first: other roundings); dx
    does not depend on the grid."""
    dn = dtype_name(dtype)
    x, dy, g, b = make_ln(outer, Rr, dtype, 43)
    rng = np.random.default_rng(44)
    dm, dv = rng.standard_normal(outer), rng.standard_normal(outer)
    _, m_r, v_r = R.ln_forward(x, b, g, outer, 1e-5)
    dx_r, dg_r, db_r = R.ln_backward(x, dy, g, m_r, v_r, outer, 1e-5, dm, dv)
    xd, dyd, gd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g)
    md, vd, dmd, dvd = to_dev(m_r), to_dev(v_r), to_dev(dm), to_dev(dv)
    try:
        K.tune_reset()
        K.tune_set("LN_BWD_BLOCKS_PER_CU", 1)
        dx, dg, db = K.ln_backward(xd, dyd, gd, md, vd, outer, 1e-5, dmean=dmd, dvar=dvd)
        K.tune_set("LN_BWD_AHEAD", 0)
        dx0, dg0, db0 = K.ln_backward(xd, dyd, gd, md, vd, outer, 1e-5, dmean=dmd, dvar=dvd)
        K.tune_reset()
        dx2, dg2, db2 = K.ln_backward(xd, dyd, gd, md, vd, outer, 1e-5, dmean=dmd, dvar=dvd)
    finally:
        K.tune_reset()
    assert_close(to_np(dx), dx_r, dn, "grad", "dx")
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")
    assert_close(to_np(dx0), to_np(dx).astype(np.float64), dn, "grad", "dx against the kernel without rows ahead")
    assert_close(to_np(dg0), to_np(dg).astype(np.float64), dn, "pgrad", "dgamma against it")
    assert_close(to_np(db0), to_np(db).astype(np.float64), dn, "pgrad", "dbeta against it")
    assert torch.equal(dx2, dx)
    assert_close(to_np(dg2), dg_r, dn, "pgrad", "dgamma, default grid")
    assert_close(to_np(db2), db_r, dn, "pgrad", "dbeta, default grid")


# Rows of 128-400 KB on at least a quarter as many rows as CUs: the forward holds
# a row on one CU (registers + LDS).  One shape per layout (10 to 25 vectors per
# thread), a row that ends inside a wave's load, several channels per row.
ONCHIP_ROWS = [
    ("in", torch.float32, 1, 64, (200, 200), 0), ("in", torch.float32, 1, 64, (216, 216), 0),
    ("in", torch.float32, 2, 32, (232, 232), 0), ("in", torch.float32, 1, 64, (250, 256), 0),
    ("in", torch.float32, 1, 64, (272, 272), 0), ("in", torch.float32, 1, 64, (296, 296), 0),
    ("in", torch.float32, 1, 64, (316, 316), 0), ("in", torch.float32, 1, 70, (2, 50002), 0),
    ("gn", torch.float32, 2, 320, (64, 64), 32), ("gn", torch.float32, 2, 512, (52, 52), 32),
    ("gn", torch.float16, 2, 640, (64, 64), 32), ("gn", torch.float16, 1, 128, (284, 284), 64),
    ("gn", torch.float16, 1, 192, (2, 2, 16666), 64), ("in", torch.float16, 1, 64, (400, 400), 0),
    ("in", torch.float16, 1, 64, (448, 446), 0), ("gn", torch.float16, 1, 1536, (90, 90), 64),
    # rows of 25601-65536 vectors: the first 25600 held, the rest streamed (forward)
    ("in", torch.float32, 1, 226, (322, 322), 0), ("gn", torch.float16, 2, 452, (2, 130004), 226),
    ("in", torch.float16, 1, 226, (2, 131076), 0),
    # InstanceNormalization backward with x of a plane held on its CU (every layout)
    ("in", torch.float32, 2, 40, (190, 190), 0), ("in", torch.float32, 1, 72, (236, 236), 0),
    ("in", torch.float32, 1, 64, (256, 256), 0), ("in", torch.float32, 1, 64, (284, 284), 0),
    ("in", torch.float16, 1, 64, (360, 360), 0), ("in", torch.float16, 2, 33, (2, 70004), 0),
    # ... with the first 18432 vectors held and the rest streamed
    ("in", torch.float32, 1, 230, (300, 300), 0), ("in", torch.float16, 1, 240, (2, 150004), 0),
    # GroupNormalization backward with the group held on its CU: x in registers and LDS,
    # dy parked in what LDS is left (10, 15, 20 and 12 vectors per thread)
    ("gn", torch.float16, 3, 960, (64, 64), 32), ("gn", torch.float32, 2, 640, (64, 64), 32),
    ("gn", torch.float16, 2, 1536, (64, 32), 64), ("gn", torch.float32, 4, 192, (64, 64), 16),
]


@pytest.mark.parametrize("kind,dtype,n,c,sp,groups", ONCHIP_ROWS)
def test_long_rows_held_on_chip(kind, dtype, n, c, sp, groups):
    dn = dtype_name(dtype)
    x, dy, g, b = make_nc(n, c, sp, dtype, 41)
    xd, gd, bd = to_dev(x, dtype), to_dev(g), to_dev(b)
    if kind == "in":
        y_r, m_r, v_r = R.in_forward(x, b, g, n, c, 1e-5)
        y, m, v = K.in_forward(xd, bd, gd, 1e-5)
    else:
        y_r, m_r, v_r = R.gn_forward(x, b, g, n, c, groups, 1e-5)
        y, m, v = K.gn_forward(xd, bd, gd, groups, 1e-5)
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(y), y_r, dn, "y", "y")
    # the backward on the statistics the forward produced
    dyd = to_dev(dy, dtype)
    if kind == "in":
        dx_r, dg_r, db_r = R.in_backward(x, dy, g, m_r, v_r, n, c, 1e-5)
        dx, dg, db = K.in_backward(xd, dyd, gd, m, v, 1e-5)
    else:
        dx_r, dg_r, db_r = R.gn_backward(x, dy, g, m_r, v_r, n, c, groups, 1e-5)
        dx, dg, db = K.gn_backward(xd, dyd, gd, m, v, groups, 1e-5)
    assert_close(to_np(dx), dx_r, dn, "grad", "dx")
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


@pytest.mark.parametrize("dtype", DTYPES)
def test_in_backward_held_on_chip_accumulate_and_parameter_gradients_only(dtype):
    dn = dtype_name(dtype)
    n, c, sp = 2, 40, ((2, 24580) if dtype == torch.float32 else (2, 49156))  # 12290 vectors
    x, dy, g, b = make_nc(n, c, sp, dtype, 43)
    _, m_r, v_r = R.in_forward(x, b, g, n, c, 1e-5)
    dx_r, dg_r, db_r = R.in_backward(x, dy, g, m_r, v_r, n, c, 1e-5)
    xd, dyd, gd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g)
    m, v = to_dev(m_r), to_dev(v_r)
    pre = rounded(np.random.default_rng(44).standard_normal(x.shape), dtype)
    dxd = to_dev(pre, dtype)
    K.in_backward(xd, dyd, gd, m, v, 1e-5, dx=dxd, accum=(True, False, False))
    assert_close(to_np(dxd), dx_r + pre, dn, "grad", "dx accumulated")
    _, dg, db = K.in_backward(xd, dyd, gd, m, v, 1e-5, need=(False, True, True))
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma only")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta only")


@pytest.mark.parametrize("n,c,sp", [(2, 8, (16, 16)), (1, 3, (300, 300)), (4, 64, (7, 7)),
                                    (1, 64, (400, 400)), (1, 226, (2, 104008)), (2, 8, (63, 63))])
def test_in_forward_in_place(n, c, sp):
    x, _, g, b = make_nc(n, c, sp, torch.float16, 32)
    y_r, m_r, v_r = R.in_forward(x, b, g, n, c, 1e-5)
    xd, gd, bd = to_dev(x, torch.float16), to_dev(g), to_dev(b)
    mean = torch.empty(n * c, device="cuda")
    var = torch.empty(n * c, device="cuda")
    L = K.lib()
    spatial = int(np.prod(sp))
    K.check(L.nblahip_in_fwd(xd.data_ptr(), gd.data_ptr(), bd.data_ptr(), xd.data_ptr(),
                             mean.data_ptr(), var.data_ptr(), n, c, spatial, 1, 1, 1e-5, 1,
                             torch.cuda.current_stream().cuda_stream))
    assert_close(to_np(xd), y_r.reshape(x.shape), "f16", "y", "y in place")
    assert_close(to_np(mean), m_r, "f16", "stat", "mean")
