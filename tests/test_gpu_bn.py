"""BatchNormalization parity on the GPU: the HIP path, called through the
C-ABI, against the float64 oracle on the same seeded inputs."""
import numpy as np
import pytest
import torch

from _util import assert_close, dtype_name, load_package, rounded, to_dev, to_np
from oracle import norm_ref as R

pytestmark = pytest.mark.gpu
K = load_package()

# (shape, axis): planes layout, channel-last, odd sizes that break 16-byte
# vectors, single-channel, sizes below one wavefront, 2-D input.
SMALL = [
    ((4, 8, 6, 6), 1), ((2, 3, 5, 7), 1), ((3, 16, 49), 1), ((5, 7), 1), ((2, 1, 9), 1),
    ((1, 4, 64, 64), 1), ((6, 5, 4, 8), 3), ((64, 64), 1), ((33, 24), 1), ((7, 3, 5, 12), 3),
    ((4, 6, 40), 2), ((2, 300, 3), 1), ((129, 5, 5, 96), 3), ((3, 2, 2, 2050), 3),
    # planes of 4k (not 8k) elements: 8-byte accesses for fp16
    ((8, 12, 14, 14), 1), ((3, 5, 4), 1), ((16, 256, 14, 14), 1),
    # planes that are no multiple of the vector width, tensor a multiple: masked vectors
    ((4, 8, 7, 7), 1), ((2, 16, 9, 9), 1), ((3, 8, 3, 11), 1), ((1, 24, 5, 5), 1),
    ((64, 32, 7, 7), 1), ((5, 16, 13), 1),
    # a channel (all its planes) in one block's registers: every row layout
    ((32, 64, 28, 28), 1), ((16, 128, 14, 14), 1), ((6, 256, 3, 3), 1), ((2, 512, 2, 2), 1),
    ((64, 40, 32, 32), 1), ((9, 33, 5, 5), 1), ((2, 64, 64, 64), 1),
    # channel-last: channel vectors that do not divide 256, rows wider than 256 vectors,
    # 8-byte fp16 rows
    ((6, 9, 9, 96), 3), ((3, 5, 5, 4104), 3), ((37, 100), 1), ((4, 6, 6, 20), 3), ((700, 1032), 1),
    # channel-last with few rows: a channel vector's column in one block's registers
    ((32, 7, 7, 512), 3), ((8, 14, 14, 256), 3), ((100, 2048), 1), ((33, 8, 8, 320), 3),
    ((5000, 256), 1), ((16, 1024), 1), ((4, 2048), 1), ((6, 64), 1),
    # tiny tensors in one launch: odd planes of 4k-8k elements per channel through
    # scalar loads, channel-last with a handful of channels as strided rows
    ((32, 64, 13, 13), 1), ((40, 5, 13, 15), 1), ((8, 14, 14, 3), 3), ((1, 64, 64, 3), 3),
    ((64, 13, 13, 3), 3), ((90, 7), 1), ((1000, 1), 1), ((2, 31, 33, 8), 3),
    # planes that are no whole number of 16-byte vectors, a pack of 2 / 4 / 8 neighbouring
    # channels per block: every slot count, samples that do not fill the last sweep, fewer
    # samples than a sweep, more samples than the backward holds, 121-vector segments,
    # pairs of half 14x14 planes (backward only)
    ((64, 1024, 7, 7), 1), ((256, 256, 7, 7), 1), ((200, 64, 14, 14), 1), ((20, 1024, 3, 3), 1),
    ((300, 256, 5, 5), 1), ((100, 264, 7, 7), 1), ((440, 256, 7, 7), 1), ((190, 512, 7, 7), 1),
    ((40, 256, 11, 11), 1),
    # channel-last through the split kernels (all rows as one plane, a unit per channel):
    # 13, 3 and 49 blocks per column tile, rows that do not fill the last block, float
    ((64, 14, 14, 128), 3), ((3000, 192), 1), ((256, 14, 14, 64), 3), ((20000, 64), 1),
    ((777, 96), 1),
    # fewer channels than CUs: a channel split over 2 / 4 / 8 blocks that exchange their sums
    # (whole and ragged last blocks, both directions in registers, LDS slots)
    ((32, 64, 56, 56), 1), ((16, 128, 56, 56), 1), ((24, 32, 48, 48), 1), ((21, 64, 40, 40), 1),
    ((32, 16, 112, 112), 1), ((64, 64, 56, 56), 1), ((84, 64, 56, 56), 1),
    # a channel per CU whose planes share cache lines with the neighbouring channels'
    ((256, 64, 14, 14), 1), ((250, 40, 10, 10), 1),
    # planes that are no whole number of vectors, a channel held by one block through the
    # tensor's aligned vectors with masked edges: one to eight vectors per thread, a
    # tensor that ends inside a vector
    ((32, 288, 35, 35), 1), ((32, 768, 17, 17), 1), ((7, 96, 17, 17), 1), ((3, 70, 9, 11), 1),
    ((64, 160, 17, 17), 1), ((5, 65, 3, 7), 1), ((40, 64, 35, 35), 1),
]
DTYPES = [torch.float32, torch.float16]


def make_bn(shape, axis, dtype, seed, mean=0.0, std=1.0):
    rng = np.random.default_rng(seed)
    c = shape[axis]
    x = rounded(rng.standard_normal(shape) * std + mean, dtype)
    dy = rounded(rng.standard_normal(shape), dtype)
    g = rng.uniform(0.5, 1.5, c).astype(np.float32).astype(np.float64)
    b = (rng.standard_normal(c) * 0.1).astype(np.float32).astype(np.float64)
    rm = (rng.standard_normal(c) * 0.1).astype(np.float32).astype(np.float64)
    rv = rng.uniform(0.5, 2.0, c).astype(np.float32).astype(np.float64)
    return x, dy, g, b, rm, rv


@pytest.mark.parametrize("shape,axis", SMALL)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("affine", [True, False])
def test_bn_inference(shape, axis, dtype, affine):
    x, _, g, b, rm, rv = make_bn(shape, axis, dtype, 0)
    if not affine:
        g = b = None
    ref = R.bn_forward_global(x, b, g, rm, rv, axis, 1e-5)
    y = K.bn_forward_global(to_dev(x, dtype), to_dev(b), to_dev(g), to_dev(rm), to_dev(rv), axis, 1e-5)
    assert_close(to_np(y), ref, dtype_name(dtype), "y", "y")


# The apply kernels keep the parameters of the channels a block meets in a
# table: planes of one vector and of 9 to 49 elements (up to a thousand planes
# per block step, vectors that straddle two planes, the wrap from the last
# channel to the first), channel-last rows of 1 to 260 vectors (column tiles
# that are not full, rows narrower than a tile).
TABLES = [
    ((70, 300, 2, 4), 1), ((33, 300, 3, 3), 1), ((16, 130, 7, 7), 1), ((40, 17, 5, 5), 1),
    ((9, 1000, 1, 8), 1), ((128, 3, 3, 5), 1), ((2, 5, 333, 8), 1),
    ((1200, 8), 1), ((700, 200), 1), ((300, 520), 1), ((150, 1000), 1), ((90, 2080), 1),
    ((64, 7, 7, 2048), 3), ((400, 133), 1),
]


@pytest.mark.parametrize("shape,axis", TABLES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tile", [None, 16, 256])
def test_bn_inference_parameter_tables(shape, axis, dtype, tile):
    if tile is not None and shape[axis] != shape[-1]:
        pytest.skip("tile width: channel-last only")
    x, _, g, b, rm, rv = make_bn(shape, axis, dtype, 3)
    ref = R.bn_forward_global(x, b, g, rm, rv, axis, 1e-5)
    if tile is not None:
        K.tune_set("BN_CL_FWD_APPLY_TILE", tile)
    try:
        y = K.bn_forward_global(to_dev(x, dtype), to_dev(b), to_dev(g), to_dev(rm), to_dev(rv), axis,
                                1e-5)
    finally:
        K.tune_reset()
    assert_close(to_np(y), ref, dtype_name(dtype), "y", "y")


@pytest.mark.parametrize("shape,axis", SMALL)
@pytest.mark.parametrize("dtype", DTYPES)
def test_bn_training_forward_backward(shape, axis, dtype):
    c = shape[axis]
    if int(np.prod(shape)) // c < 2:
        pytest.skip("N == 1")
    dn = dtype_name(dtype)
    x, dy, g, b, rm, rv = make_bn(shape, axis, dtype, 1, mean=1.0, std=2.0)
    y_r, m_r, v_r, rm_r, rv_r = R.bn_forward_batch(x, b, g, rm, rv, axis, 0.9, 1e-5)
    dx_r, dg_r, db_r = R.bn_backward_batch(x, dy, g, m_r, v_r, axis, 1e-5)

    xd, dyd, gd, bd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(b)
    rmd, rvd = to_dev(rm), to_dev(rv)
    y, m, v = K.bn_forward_batch(xd, bd, gd, rmd, rvd, axis, 0.9, 1e-5)
    assert_close(to_np(y), y_r, dn, "y", "y")
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(rmd), rm_r, dn, "stat", "running_mean")
    assert_close(to_np(rvd), rv_r, dn, "stat", "running_var")
    dx, dg, db = K.bn_backward(xd, dyd, gd, m, v, axis, 1e-5)
    assert_close(to_np(dx), dx_r, dn, "grad", "dx")
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


@pytest.mark.parametrize("shape,axis", [((4, 8, 6, 6), 1), ((37, 24), 1), ((6, 5, 4, 8), 3),
                                        # a channel per block, cached in registers
                                        ((8, 64, 12, 12), 1), ((4, 48, 7, 9), 1), ((3, 300, 2, 2), 1),
                                        # a pack of channels per block (planes of 49 elements)
                                        ((90, 256, 7, 7), 1),
                                        # odd planes, a channel held by one block
                                        ((6, 80, 17, 17), 1),
                                        # a channel split over 4 blocks
                                        ((40, 64, 32, 32), 1),
                                        # channel-last through the split kernels
                                        ((40, 14, 14, 64), 3),
                                        # channel-last, a channel vector's column per block
                                        ((8, 7, 7, 256), 3), ((300, 512), 1)])
def test_bn_flags(shape, axis):
    """no_scale/no_bias, recompute (no running update), accumulation,
    propagate_down subsets, 3-output dmean/dvar."""
    dtype = torch.float32
    c = shape[axis]
    x, dy, g, b, rm, rv = make_bn(shape, axis, dtype, 2)
    rng = np.random.default_rng(3)
    dm, dv = rng.standard_normal(c), rng.standard_normal(c)
    xd, dyd = to_dev(x), to_dev(dy)

    # no_scale / no_bias and recompute_impl (running stats untouched = NULL)
    y_r, m_r, v_r, _, _ = R.bn_forward_batch(x, None, None, None, None, axis, 0.9, 1e-5)
    y, m, v = K.bn_forward_batch(xd, None, None, None, None, axis, 0.9, 1e-5)
    assert_close(to_np(y), y_r, "f32", "y", "y no affine")
    dx_r, dg_r, db_r = R.bn_backward_batch(x, dy, None, m_r, v_r, axis, 1e-5, dm, dv)
    dx, dg, db = K.bn_backward(xd, dyd, None, m, v, axis, 1e-5, dmean=to_dev(dm), dvar=to_dev(dv))
    assert_close(to_np(dx), dx_r, "f32", "grad", "dx 3-output")
    assert_close(to_np(dg), dg_r, "f32", "pgrad", "dgamma")
    assert_close(to_np(db), db_r, "f32", "pgrad", "dbeta")

    # accumulation onto existing gradients, gamma present
    _, m_r, v_r, _, _ = R.bn_forward_batch(x, b, g, None, None, axis, 0.9, 1e-5)
    dx_r, dg_r, db_r = R.bn_backward_batch(x, dy, g, m_r, v_r, axis, 1e-5)
    pre_dx = rng.standard_normal(shape).astype(np.float32)
    pre_g = rng.standard_normal(c).astype(np.float32)
    pre_b = rng.standard_normal(c).astype(np.float32)
    dxd, dgd, dbd = to_dev(pre_dx), to_dev(pre_g), to_dev(pre_b)
    K.bn_backward(xd, dyd, to_dev(g), to_dev(m_r), to_dev(v_r), axis, 1e-5, dx=dxd, dgamma=dgd,
                  dbeta=dbd, accum=(True, True, True))
    assert_close(to_np(dxd), dx_r + pre_dx, "f32", "grad", "dx accum")
    assert_close(to_np(dgd), dg_r + pre_g, "f32", "pgrad", "dgamma accum")
    assert_close(to_np(dbd), db_r + pre_b, "f32", "pgrad", "dbeta accum")

    # propagate_down subsets: only parameters / only dx
    sentinel = to_dev(np.full(shape, 7.0, np.float32))
    _, dg, db = K.bn_backward(xd, dyd, to_dev(g), to_dev(m_r), to_dev(v_r), axis, 1e-5,
                              need=(False, True, True))
    assert_close(to_np(dg), dg_r, "f32", "pgrad", "dgamma only")
    assert_close(to_np(db), db_r, "f32", "pgrad", "dbeta only")
    dx, _, _ = K.bn_backward(xd, dyd, to_dev(g), to_dev(m_r), to_dev(v_r), axis, 1e-5, dx=sentinel,
                             need=(True, False, False))
    assert_close(to_np(dx), dx_r, "f32", "grad", "dx only")


@pytest.mark.parametrize("shape,axis", [((4, 8, 6, 6), 1), ((6, 5, 4, 8), 3)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_bn_inference_mode_backward(shape, axis, dtype):
    dn = dtype_name(dtype)
    x, dy, g, b, rm, rv = make_bn(shape, axis, dtype, 4)
    dx_r, dg_r, db_r = R.bn_backward_global(x, dy, g, rm, rv, axis, 1e-5)
    dx, dg, db = K.bn_backward(to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(rm),
                               to_dev(rv), axis, 1e-5, batch_stat=False)
    assert_close(to_np(dx), dx_r, dn, "grad", "dx")
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


def test_bn_constant_input_and_determinism():
    x = torch.full((8, 16, 14, 14), 2.5, device="cuda")
    b = torch.linspace(-1, 1, 16, device="cuda")
    y, m, v = K.bn_forward_batch(x, b, torch.ones(16, device="cuda"), None, None, 1, 0.9, 1e-5)
    assert torch.equal(v, torch.zeros_like(v))
    assert torch.equal(y, b.view(1, 16, 1, 1).expand_as(x).contiguous())
    xr = torch.randn(16, 32, 28, 28, device="cuda")
    a1 = K.bn_forward_batch(xr, None, None, None, None, 1, 0.9, 1e-5)
    a2 = K.bn_forward_batch(xr, None, None, None, None, 1, 0.9, 1e-5)
    for p, q in zip(a1, a2):
        assert torch.equal(p, q)


def test_bn_misaligned_views():
    """Pointers that are not 16-byte aligned take the scalar-load plan."""
    rng = np.random.default_rng(5)
    shape, axis = (4, 8, 6, 6), 1
    n = int(np.prod(shape))
    x = rng.standard_normal(n + 1).astype(np.float32)
    xd = to_dev(x)[1:].view(shape)
    assert xd.data_ptr() % 16 != 0
    xs = x[1:].reshape(shape).astype(np.float64)
    y_r, m_r, v_r, _, _ = R.bn_forward_batch(xs, None, None, None, None, axis, 0.9, 1e-5)
    y, m, v = K.bn_forward_batch(xd, None, None, None, None, axis, 0.9, 1e-5)
    assert_close(to_np(y), y_r, "f32", "y", "y")
    assert_close(to_np(v), v_r, "f32", "stat", "var")


@pytest.mark.parametrize("dtype", DTYPES)
def test_bn_odd_planes_channel_owning_blocks(dtype):
    """33x33 planes (no multiple of the vector width) with enough data per
    channel for the blocks that own a whole channel."""
    dn = dtype_name(dtype)
    shape, axis = (128, 256, 33, 33), 1
    x, dy, g, b, rm, rv = make_bn(shape, axis, dtype, 17, mean=0.5, std=1.5)
    y_r, m_r, v_r, rm_r, rv_r = R.bn_forward_batch(x, b, g, rm, rv, axis, 0.9, 1e-5)
    xd, dyd, gd, bd, rmd, rvd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(b), to_dev(rm), to_dev(rv)
    y, m, v = K.bn_forward_batch(xd, bd, gd, rmd, rvd, axis, 0.9, 1e-5)
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(rvd), rv_r, dn, "stat", "running_var")
    assert_close(to_np(y), y_r, dn, "y", "y")
    del y_r
    dx_r, dg_r, db_r = R.bn_backward_batch(x, dy, g, m_r, v_r, axis, 1e-5)
    dx, dg, db = K.bn_backward(xd, dyd, gd, m, v, axis, 1e-5)
    assert_close(to_np(dx), dx_r, dn, "grad", "dx")
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


def test_bn_c1_inference_full_size():
    """Benchmark configuration 1: x[8,64,56,56] fp32, inference, seed 0."""
    rng = np.random.default_rng(0)
    shape = (8, 64, 56, 56)
    x = rng.standard_normal(shape).astype(np.float32)
    g = rng.uniform(0.5, 1.5, 64).astype(np.float32)
    b = (rng.standard_normal(64) * 0.1).astype(np.float32)
    rm = (rng.standard_normal(64) * 0.1).astype(np.float32)
    rv = rng.uniform(0.5, 2, 64).astype(np.float32)
    ref = R.bn_forward_global(x, b, g, rm, rv, 1, 1e-5)
    y = K.bn_forward_global(to_dev(x), to_dev(b), to_dev(g), to_dev(rm), to_dev(rv), 1, 1e-5)
    assert_close(to_np(y), ref, "f32", "y", "y")


def test_bn_c2_training_full_size():
    """Benchmark configuration 2: x[32,256,56,56] ~ N(1,2) fp32, fwd+bwd, seed 1."""
    rng = np.random.default_rng(1)
    shape = (32, 256, 56, 56)
    x = (rng.standard_normal(shape, dtype=np.float32) * 2 + 1).astype(np.float32)
    dy = rng.standard_normal(shape, dtype=np.float32)
    g = rng.uniform(0.5, 1.5, 256).astype(np.float32)
    b = (rng.standard_normal(256) * 0.1).astype(np.float32)
    rm = np.zeros(256, np.float32)
    rv = np.ones(256, np.float32)
    y_r, m_r, v_r, rm_r, rv_r = R.bn_forward_batch(x, b, g, rm, rv, 1, 0.9, 1e-5)
    dx_r, dg_r, db_r = R.bn_backward_batch(x, dy, g, m_r, v_r, 1, 1e-5)
    xd, dyd, gd, bd, rmd, rvd = map(to_dev, (x, dy, g, b, rm, rv))
    y, m, v = K.bn_forward_batch(xd, bd, gd, rmd, rvd, 1, 0.9, 1e-5)
    dx, dg, db = K.bn_backward(xd, dyd, gd, m, v, 1, 1e-5)
    assert_close(to_np(y), y_r, "f32", "y", "y")
    assert_close(to_np(m), m_r, "f32", "stat", "mean")
    assert_close(to_np(v), v_r, "f32", "stat", "var")
    assert_close(to_np(rmd), rm_r, "f32", "stat", "running_mean")
    assert_close(to_np(rvd), rv_r, "f32", "stat", "running_var")
    assert_close(to_np(dx), dx_r, "f32", "grad", "dx")
    assert_close(to_np(dg), dg_r, "f32", "pgrad", "dgamma")
    assert_close(to_np(db), db_r, "f32", "pgrad", "dbeta")
    # size-independent invariants of the batch backward
    dxn = to_np(dx).reshape(32, 256, -1)
    assert np.abs(dxn.sum(axis=(0, 2))).max() < 1e-2


def test_bn_c5_channel_last_fp16_full_size():
    """Benchmark configuration 5: x[256,56,56,64] fp16 with 1% outliers x50, axes=[3],
    fp32 statistics, split reduction over 802816 rows, seed 4."""
    rng = np.random.default_rng(4)
    shape = (256, 56, 56, 64)
    x = rng.standard_normal(shape, dtype=np.float32)
    mask = rng.random(shape, dtype=np.float32) < 0.01
    x = np.where(mask, x * 50, x).astype(np.float16)
    del mask
    dy = rng.standard_normal(shape, dtype=np.float32).astype(np.float16)
    g = rng.uniform(0.5, 1.5, 64).astype(np.float32)
    b = (rng.standard_normal(64) * 0.1).astype(np.float32)
    rm = np.zeros(64, np.float32)
    rv = np.ones(64, np.float32)
    xd, dyd = torch.from_numpy(x).cuda(), torch.from_numpy(dy).cuda()
    gd, bd, rmd, rvd = map(to_dev, (g, b, rm, rv))
    y, m, v = K.bn_forward_batch(xd, bd, gd, rmd, rvd, 3, 0.9, 1e-5)
    dx, dg, db = K.bn_backward(xd, dyd, gd, m, v, 3, 1e-5)
    torch.cuda.synchronize()
    y_r, m_r, v_r, rm_r, rv_r = R.bn_forward_batch(x, b, g, rm, rv, 3, 0.9, 1e-5)
    assert_close(to_np(m), m_r, "f16", "stat", "mean")
    assert_close(to_np(v), v_r, "f16", "stat", "var")
    assert_close(to_np(rmd), rm_r, "f16", "stat", "running_mean")
    assert_close(to_np(rvd), rv_r, "f16", "stat", "running_var")
    assert_close(to_np(y), y_r, "f16", "y", "y")
    del y_r
    dx_r, dg_r, db_r = R.bn_backward_batch(x, dy, g, m_r, v_r, 3, 1e-5)
    assert_close(to_np(dx), dx_r, "f16", "grad", "dx")
    assert_close(to_np(dg), dg_r, "f16", "pgrad", "dgamma")
    assert_close(to_np(db), db_r, "f16", "pgrad", "dbeta")


def test_bn_argument_errors():
    x = torch.randn(4, 8, 6, 6, device="cuda")
    L = K.lib()
    s = torch.cuda.current_stream().cuda_stream
    m = torch.empty(8, device="cuda")
    y = torch.empty_like(x)
    # unknown dtype
    assert L.nblahip_bn_fwd_infer(x.data_ptr(), m.data_ptr(), m.data_ptr(), None, None,
                                  y.data_ptr(), 4, 8, 36, 1e-5, 7, s) == -1
    # missing required pointer
    assert L.nblahip_bn_fwd_infer(None, m.data_ptr(), m.data_ptr(), None, None, y.data_ptr(), 4, 8,
                                  36, 1e-5, 0, s) == -1
    # workspace too small / missing
    assert L.nblahip_bn_fwd_train(x.data_ptr(), None, None, y.data_ptr(), m.data_ptr(),
                                  m.data_ptr(), None, None, 4, 8, 36, 0.9, 1e-5, 0, None, 0, s) == -2
    # negative size
    assert L.nblahip_bn_fwd_infer(x.data_ptr(), m.data_ptr(), m.data_ptr(), None, None,
                                  y.data_ptr(), -1, 8, 36, 1e-5, 0, s) == -1
    # empty tensor: success, nothing launched
    assert L.nblahip_bn_fwd_infer(x.data_ptr(), m.data_ptr(), m.data_ptr(), None, None,
                                  y.data_ptr(), 0, 8, 36, 1e-5, 0, s) == 0
    with pytest.raises(K.NblaHipError):
        K.check(-3)


# A channel held on one CU (registers, then LDS): needs a channel for (nearly)
# every CU and 8193 to 25600 vectors per channel.  N picks the vectors per
# thread (9 to 25), hence the register/LDS layout; odd N leaves the last slot
# partly filled.  Backward layouts that hold the whole channel end at 20480
# vectors (the last one with 512 threads per block); beyond, 18432 are held,
# the next 3072 parked in LDS by the first pass, and the rest is streamed.
ONCHIP_CASES = [(torch.float32, 33), (torch.float32, 47), (torch.float32, 55), (torch.float32, 63),
                (torch.float32, 71), (torch.float32, 77), (torch.float32, 85), (torch.float32, 99),
                (torch.float16, 67), (torch.float16, 111), (torch.float16, 141),
                (torch.float16, 155), (torch.float16, 197),
                # longer than the chip holds: 25600 (forward) / 18432 (backward) vectors
                # stay, the rest is streamed
                (torch.float32, 131), (torch.float16, 301),
                # ... with a remainder short enough for the LDS the held slots leave
                # free (3072 vectors, parked during the backward's first pass)
                (torch.float32, 83), (torch.float16, 165), (torch.float32, 84)]


@pytest.mark.parametrize("dtype,n", ONCHIP_CASES)
@pytest.mark.parametrize("few_channels", [False, True])
def test_bn_channel_on_chip(dtype, n, few_channels):
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    # a channel for (nearly) every CU, or for a quarter of them (whole-channel
    # layouts only; the others then take the split reduction)
    c = (cus + 3) // 4 + 1 if few_channels else (cus * 7 + 7) // 8
    check_channel_on_chip((n, c, 32, 32), dtype)


# Half planes of 4k (not 8k) elements (14 x 14) are held as 8-byte vectors, up
# to 16384 of them per channel (the last shape is beyond: split reduction).
@pytest.mark.parametrize("shape", [(180, 64, 14, 14), (330, 72, 14, 14), (420, 72, 14, 14)])
def test_bn_channel_on_chip_8_byte_vectors(shape):
    check_channel_on_chip(shape, torch.float16)


def check_channel_on_chip(shape, dtype):
    axis, c = 1, shape[1]
    dn = dtype_name(dtype)
    x, dy, g, b, rm, rv = make_bn(shape, axis, dtype, 21, mean=1.0, std=2.0)
    y_r, m_r, v_r, rm_r, rv_r = R.bn_forward_batch(x, b, g, rm, rv, axis, 0.9, 1e-5)
    rng = np.random.default_rng(22)
    dm, dv = rng.standard_normal(c), rng.standard_normal(c)
    dx_r, dg_r, db_r = R.bn_backward_batch(x, dy, g, m_r, v_r, axis, 1e-5, dm, dv)
    xd, dyd, gd, bd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(b)
    rmd, rvd = to_dev(rm), to_dev(rv)
    y, m, v = K.bn_forward_batch(xd, bd, gd, rmd, rvd, axis, 0.9, 1e-5)
    assert_close(to_np(y), y_r, dn, "y", "y")
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(rmd), rm_r, dn, "stat", "running_mean")
    assert_close(to_np(rvd), rv_r, dn, "stat", "running_var")
    if dtype == torch.float32:  # accumulated onto an existing gradient
        pre = torch.randn_like(xd)
        dx, dg, db = K.bn_backward(xd, dyd, gd, m, v, axis, 1e-5, dmean=to_dev(dm), dvar=to_dev(dv),
                                   dx=pre.clone(), accum=(True, False, False))
        assert_close(to_np(dx) - to_np(pre), dx_r, dn, "grad", "dx (accumulated)")
    else:
        dx, dg, db = K.bn_backward(xd, dyd, gd, m, v, axis, 1e-5, dmean=to_dev(dm), dvar=to_dev(dv))
        assert_close(to_np(dx), dx_r, dn, "grad", "dx")
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")
    # run to run, and without dx
    y2, _, _ = K.bn_forward_batch(xd, bd, gd, to_dev(rm), to_dev(rv), axis, 0.9, 1e-5)
    assert torch.equal(y2, y)
    _, dg2, db2 = K.bn_backward(xd, dyd, gd, m, v, axis, 1e-5, need=(False, True, True))
    assert torch.equal(dg2, dg) and torch.equal(db2, db)


@pytest.mark.parametrize("shape,axis,dtype", [
    ((8, 12, 14, 14), 1, torch.float32),      # split reduction
    ((8, 64, 12, 12), 1, torch.float32),      # channel in one block's registers
    ((9, 72, 17, 17), 1, torch.float16),      # odd planes, a channel held by one block
    ((37, 64, 32, 32), 1, torch.float32),     # channel held on one CU
    ((131, 232, 16, 32), 1, torch.float16),   # ... with a streamed remainder
    ((8, 7, 7, 256), 3, torch.float16),       # channel-last, column in registers
    ((300, 9, 64), 2, torch.float32),         # channel-last split reduction
])
def test_bn_training_forward_in_place(shape, axis, dtype):
    """y == x through the C-ABI on every forward path."""
    dn = dtype_name(dtype)
    x, _, g, b, rm, rv = make_bn(shape, axis, dtype, 33, mean=0.5, std=1.5)
    y_r, m_r, v_r, rm_r, rv_r = R.bn_forward_batch(x, b, g, rm, rv, axis, 0.9, 1e-5)
    xd, gd, bd, rmd, rvd = to_dev(x, dtype), to_dev(g), to_dev(b), to_dev(rm), to_dev(rv)
    c = shape[axis]
    m, v = torch.empty(c, device="cuda"), torch.empty(c, device="cuda")
    s0, _, s2 = K._bn_sizes(shape, axis)
    L = K.lib()
    dt = K._dtype_code(xd)
    ws = torch.empty(max(int(L.nblahip_bn_workspace_bytes(s0, c, s2, dt)), 256), dtype=torch.uint8,
                     device="cuda")
    K.check(L.nblahip_bn_fwd_train(xd.data_ptr(), gd.data_ptr(), bd.data_ptr(), xd.data_ptr(),
                                   m.data_ptr(), v.data_ptr(), rmd.data_ptr(), rvd.data_ptr(), s0, c,
                                   s2, 0.9, 1e-5, dt, ws.data_ptr(), ws.numel(),
                                   torch.cuda.current_stream().cuda_stream))
    assert_close(to_np(xd), y_r, dn, "y", "y in place")
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(rmd), rm_r, dn, "stat", "running_mean")


# ------------------------------------------------------------------
# Channel-last training forward with the whole tensor held on the chip and the
# per-channel partials exchanged between the blocks.
@pytest.mark.parametrize("m,c,dtype", [(100352, 64, torch.float16), (100353, 64, torch.float16),
                                       (200000, 32, torch.float32), (150000, 128, torch.float16),
                                       (1000001, 8, torch.float16), (40000, 128, torch.float32),
                                       # more than 128 channels: column strips, a block merges several channels
                                       (40000, 256, torch.float16), (50000, 512, torch.float16),
                                       (40000, 256, torch.float32),
                                       # 8 and 16 strips; 3 strips of 64 channels (255 blocks); strips of 32 channels
                                       (20001, 1024, torch.float16), (9000, 2048, torch.float32),
                                       (40000, 192, torch.float16), (37000, 96, torch.float32),
                                       (12345, 4096, torch.float16)])
def test_bn_channel_last_held_on_the_chip(m, c, dtype):
    """Against the oracle; bit-identical when no poll is allowed (every block
    then computes the partials and channel results it needs itself); close to
    the split reduction; running statistics updated once."""
    _held_forward(m, c, dtype, {})


# Fewer blocks than CUs, so that a small tensor is more than the blocks hold:
# 47 and 59 vectors per thread (25 held), with one strip, with three, in float.
@pytest.mark.parametrize("m,c,dtype,blocks", [(48000, 128, torch.float16, 16), (24001, 384, torch.float16, 24),
                                              (40000, 64, torch.float32, 16), (60000, 128, torch.float16, 16)])
def test_bn_channel_last_more_than_the_chip_holds(m, c, dtype, blocks):
    """What the blocks do not hold is read for the statistics and again for
    the normalization; same checks as with everything held."""
    _held_forward(m, c, dtype, {"BN_CL_GRID_BLOCKS": blocks, "BN_CL_GRID_WIDE_MIN_KB": 1})


def _held_forward(m, c, dtype, extra):
    dn = dtype_name(dtype)
    x, _, g, b, rm, rv = make_bn((m, c), 1, dtype, 5, mean=1.0, std=2.0)
    y_r, m_r, v_r, rm_r, rv_r = R.bn_forward_batch(x, b, g, rm, rv, 1, 0.9, 1e-5)
    xd, gd, bd = to_dev(x, dtype), to_dev(g), to_dev(b)

    def run(knobs):
        K.tune_reset()
        for k_, val in knobs.items():
            K.tune_set(k_, val)
        rmd, rvd = to_dev(rm), to_dev(rv)
        K.check(K.lib().nblahip_profile_enable(16))
        y, mean, var = K.bn_forward_batch(xd, bd, gd, rmd, rvd, 1, 0.9, 1e-5)
        torch.cuda.synchronize()
        names = K.profile_kernels()
        K.check(K.lib().nblahip_profile_enable(0))
        K.tune_reset()
        return [y, mean, var, rmd, rvd], names

    try:
        held, names = run({**extra, "BN_CL_GRID_MIN_SLOTS": 1})
        assert names == ["bn_cl_grid_fwd_kernel"], names
        alone, names = run({**extra, "BN_CL_GRID_MIN_SLOTS": 1, "XCHG_SPIN": 0})
        assert names == ["bn_cl_grid_fwd_kernel"], names
        split, names = run({"BN_CL_GRID": 0})
        assert "bn_cl_grid_fwd_kernel" not in names
    finally:
        K.tune_reset()
    y, mean, var, rmd, rvd = held
    assert_close(to_np(mean), m_r, dn, "stat", "mean")
    assert_close(to_np(var), v_r, dn, "stat", "var")
    assert_close(to_np(rmd), rm_r, dn, "stat", "running mean")
    assert_close(to_np(rvd), rv_r, dn, "stat", "running var")
    assert_close(to_np(y), y_r, dn, "y", "y")
    for a_, b_ in zip(held, alone):
        assert torch.equal(a_, b_)
    assert_close(to_np(split[0]), to_np(y), dn, "y", "y against the split reduction")
    assert_close(to_np(split[2]), to_np(var), dn, "stat", "var against the split reduction")


@pytest.mark.parametrize("m,c,dtype", [(100352, 64, torch.float16), (100353, 64, torch.float16),
                                       (200000, 32, torch.float32), (150000, 128, torch.float16),
                                       (1000001, 8, torch.float16), (40000, 128, torch.float32),
                                       # more of x than a block holds: the rest is read again
                                       (750000, 64, torch.float16), (380000, 64, torch.float32),
                                       # 256 and 512 channels (column strips); more than the 21 vectors held
                                       (40000, 256, torch.float16), (50000, 512, torch.float16),
                                       (40000, 256, torch.float32), (170000, 256, torch.float16),
                                       # column strips: 8 and 16 of them; 3 of 64 channels; of 32 channels;
                                       # 32 of them; more of x than the blocks of a strip hold
                                       (20001, 1024, torch.float16), (9000, 2048, torch.float32),
                                       (40000, 192, torch.float16), (37000, 96, torch.float32),
                                       (12345, 4096, torch.float16), (46000, 1024, torch.float16)])
def test_bn_channel_last_backward_held_on_the_chip(m, c, dtype):
    """Backward with x held on the chip and the (sum dy*xh, sum dy) pairs
    exchanged: against the oracle with the 3-output terms, bit-identical when no
    poll is allowed, close to the split reduction; accumulation and the
    parameters-only call."""
    _held_backward(m, c, dtype, {})


@pytest.mark.parametrize("m,c,dtype,blocks", [(48000, 128, torch.float16, 16), (24001, 384, torch.float16, 24),
                                              (40000, 64, torch.float32, 16)])
def test_bn_channel_last_backward_more_than_the_chip_holds(m, c, dtype, blocks):
    """40 and 47 vectors per thread, 21 of x held: the rest streamed two at a time."""
    _held_backward(m, c, dtype, {"BN_CL_GRID_BLOCKS": blocks, "BN_CL_GRID_WIDE_MIN_KB": 1})


def _held_backward(m, c, dtype, extra):
    dn = dtype_name(dtype)
    x, dy, g, b, _, _ = make_bn((m, c), 1, dtype, 6, mean=1.0, std=2.0)
    rng = np.random.default_rng(7)
    dm, dv = rng.standard_normal(c), rng.standard_normal(c)
    _, m_r, v_r, _, _ = R.bn_forward_batch(x, b, g, None, None, 1, 0.9, 1e-5)
    dx_r, dg_r, db_r = R.bn_backward_batch(x, dy, g, m_r, v_r, 1, 1e-5, dm, dv)
    xd, dyd, gd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g)
    md, vd, dmd, dvd = to_dev(m_r), to_dev(v_r), to_dev(dm), to_dev(dv)
    pre_dx = rounded(rng.standard_normal((m, c)), dtype)
    pre_g, pre_b = rng.standard_normal(c), rng.standard_normal(c)

    def run(knobs, **kw):
        K.tune_reset()
        for k_, val in knobs.items():
            K.tune_set(k_, val)
        K.check(K.lib().nblahip_profile_enable(16))
        out = K.bn_backward(xd, dyd, gd, md, vd, 1, 1e-5, dmean=dmd, dvar=dvd, **kw)
        torch.cuda.synchronize()
        names = K.profile_kernels()
        K.check(K.lib().nblahip_profile_enable(0))
        K.tune_reset()
        return out, names

    try:
        held, names = run({**extra, "BN_CL_GRID_MIN_SLOTS": 1})
        assert names == ["bn_cl_grid_bwd_kernel"], names
        alone, names = run({**extra, "BN_CL_GRID_MIN_SLOTS": 1, "XCHG_SPIN": 0})
        assert names == ["bn_cl_grid_bwd_kernel"], names
        split, names = run({"BN_CL_GRID_BWD": 0, "BN_CL_GRID_MIN_SLOTS": 1})
        assert "bn_cl_grid_bwd_kernel" not in names
        acc, names = run({**extra, "BN_CL_GRID_MIN_SLOTS": 1}, dx=to_dev(pre_dx, dtype), dgamma=to_dev(pre_g),
                         dbeta=to_dev(pre_b), accum=(True, True, True))
        assert names == ["bn_cl_grid_bwd_kernel"], names
        params, names = run({**extra, "BN_CL_GRID_MIN_SLOTS": 1}, need=(False, True, True))
        assert names == ["bn_cl_grid_bwd_kernel"], names
    finally:
        K.tune_reset()
    dx, dg, db = held
    assert_close(to_np(dx), dx_r, dn, "grad", "dx")
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")
    for a_, b_ in zip(held, alone):
        assert torch.equal(a_, b_)
    assert_close(to_np(split[0]), to_np(dx), dn, "grad", "dx against the split reduction")
    assert_close(to_np(split[1]), to_np(dg), dn, "pgrad", "dgamma against the split reduction")
    assert_close(to_np(acc[0]), dx_r + pre_dx, dn, "grad", "dx accumulated")
    assert_close(to_np(acc[1]), dg_r + pre_g, dn, "pgrad", "dgamma accumulated")
    assert_close(to_np(acc[2]), db_r + pre_b, dn, "pgrad", "dbeta accumulated")
    assert params[0] is None
    assert torch.equal(params[1], dg) and torch.equal(params[2], db)


@pytest.mark.parametrize("kind", ["offset", "outlier_first", "constant"])
@pytest.mark.parametrize("shape,axis,dtype,kernel,knobs", [
    ((32, 64, 56, 56), 1, torch.float32, "bn_onchip_fwd_kernel", {"BN_CHAN_SPLIT": 0}),
    ((32, 64, 56, 56), 1, torch.float16, "bn_onchip_fwd_kernel", {"BN_CHAN_SPLIT": 0}),
    ((32, 64, 56, 56), 1, torch.float32, "bn_chan_split_fwd_kernel", {}),
    ((32, 64, 56, 56), 1, torch.float16, "bn_chan_split_fwd_kernel", {}),
    ((150000, 64), 1, torch.float32, "bn_cl_grid_fwd_kernel", {"BN_CL_GRID_MIN_SLOTS": 1}),
    ((150000, 64), 1, torch.float16, "bn_cl_grid_fwd_kernel", {"BN_CL_GRID_MIN_SLOTS": 1}),
    # (more than the blocks hold: the streamed part is taken about the mean of the part held)
    ((48000, 128), 1, torch.float16, "bn_cl_grid_fwd_kernel", {"BN_CL_GRID_MIN_SLOTS": 1, "BN_CL_GRID_BLOCKS": 16}),
    ((40000, 64), 1, torch.float32, "bn_cl_grid_fwd_kernel", {"BN_CL_GRID_MIN_SLOTS": 1, "BN_CL_GRID_BLOCKS": 16}),
    ((200, 256, 7, 7), 1, torch.float32, "bn_pack_fwd_kernel", {}),
    ((200, 384, 7, 7), 1, torch.float16, "bn_pack_fwd_kernel", {}),
    ((12000, 128), 1, torch.float16, "cl_split_fwd_kernel", {"BN_CL_GRID": 0}),
])
def test_one_pass_statistics_on_hard_data(kind, shape, axis, dtype, kernel, knobs):
    """The statistics shift by each thread's own mean: a mean far
    from zero, one huge value in the very first element of every channel (1000
    deviations off everything else its thread holds), and constant data
    (variance 0 to rounding) must all come out within the statistics' tolerance."""
    dn = dtype_name(dtype)
    rng = np.random.default_rng(77)
    c = shape[axis]
    if kind == "offset":
        x = rng.standard_normal(shape) + (300.0 if dtype == torch.float32 else 40.0)
    elif kind == "outlier_first":
        x = rng.standard_normal(shape)
        first = [0] * len(shape)
        first[axis] = slice(None)
        x[tuple(first)] = 1000.0
    else:
        x = np.full(shape, 3.25)
    x = rounded(x, dtype)
    y_r, m_r, v_r, _, _ = R.bn_forward_batch(x, None, None, None, None, axis, 0.9, 1e-5)
    for name, value in knobs.items():
        K.tune_set(name, value)
    try:
        K.check(K.lib().nblahip_profile_enable(8))
        y, m, v = K.bn_forward_batch(to_dev(x, dtype), None, None, None, None, axis, 0.9, 1e-5)
        torch.cuda.synchronize()
        assert K.profile_kernels() == [kernel]
    finally:
        K.check(K.lib().nblahip_profile_enable(0))
        K.tune_reset()
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    if kind == "constant":
        assert float(v.abs().max()) < 1e-10
    # (at an offset of 300 a float x is itself only known to 3e-5, and so is x - mean)
    assert_close(to_np(y), y_r, dn, "y", "y",
                 scale=10.0 if kind == "offset" and dtype == torch.float32 else 1.0 if kind == "constant" else None)


def test_two_chip_filling_forwards_at_once():
    """Two host threads, each on its own stream, run the forward that holds the
    whole tensor on the chip at the same time: each launch wants every CU, so
    blocks of the two launches wait for partners that are not resident yet, time
    out and compute what they need themselves.  Both must finish and give the
    single-threaded results bit for bit."""
    import threading
    m, c = 256 * 56 * 56, 64

    def work(seed, reps):
        gen = torch.Generator(device="cuda").manual_seed(seed)
        x = (torch.randn(m, c, device="cuda", generator=gen) * 2 + 1).half()
        gamma = torch.rand(c, device="cuda", generator=gen) + 0.5
        beta = torch.randn(c, device="cuda", generator=gen)
        out = None
        for _ in range(reps):
            out = K.bn_forward_batch(x, beta, gamma, None, None, 1, 0.9, 1e-5)
        return list(out)

    K.check(K.lib().nblahip_profile_enable(8))
    want = [[t.clone() for t in work(300 + i, 1)] for i in range(2)]
    torch.cuda.synchronize()
    assert K.profile_kernels() == ["bn_cl_grid_fwd_kernel"]
    K.check(K.lib().nblahip_profile_enable(0))
    got, errors = [None, None], []

    def run(i):
        try:
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                out = work(300 + i, 4)
                s.synchronize()
            got[i] = out
        except Exception as e:  # noqa: BLE001 - reported below
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=run, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for w, g_ in zip(want, got):
        for a_, b_ in zip(w, g_):
            assert torch.equal(a_, b_)
