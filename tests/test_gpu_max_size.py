"""Tensors just below 2^31 elements (fp16, 4.3 GB each), the most one launch
indexes, and just above, where the C-ABI runs ranges: the 32-bit index
arithmetic of the kernels must not wrap.  The input is a small
block tiled along the batch, so every tile must reproduce the result of the
block alone, which the float64 oracle checks; parameter gradients scale with
the number of tiles."""
import numpy as np
import pytest
import torch

from _util import assert_close, load_package, to_dev, to_np
from oracle import norm_ref as R

pytestmark = pytest.mark.gpu
K = load_package()


def _need(gib):
    free, _ = torch.cuda.mem_get_info()
    if free < gib * (1 << 30):
        pytest.skip(f"needs {gib} GiB of free device memory")


def test_layer_normalization_just_below_2_31_elements():
    _need(24)
    Rr, blk = 8192, 64
    tiles = ((1 << 31) - 1) // (Rr * blk)            # 4095 tiles -> 2 146 959 360 elements
    rows = tiles * blk
    assert rows * Rr < (1 << 31) and rows * Rr > (1 << 31) - (1 << 21)
    rng = np.random.default_rng(61)
    xb = (rng.standard_normal((blk, Rr)) + rng.uniform(-3, 3, (blk, 1))).astype(np.float16)
    dyb = rng.standard_normal((blk, Rr)).astype(np.float16)
    g = (rng.standard_normal(Rr) * 0.1 + 1).astype(np.float32)
    b = (rng.standard_normal(Rr) * 0.1).astype(np.float32)
    x = torch.from_numpy(xb).cuda().repeat(tiles, 1)
    dy = torch.from_numpy(dyb).cuda().repeat(tiles, 1)
    gd, bd = to_dev(g), to_dev(b)
    y, m, v = K.ln_forward(x, bd, gd, rows, 1e-5)
    y_r, m_r, v_r = R.ln_forward(xb, b, g, blk, 1e-5)
    assert_close(to_np(y[:blk]), y_r, "f16", "y", "first tile y")
    assert_close(to_np(m[:blk]), m_r, "f16", "stat", "first tile mean")
    yt = y.view(tiles, blk, Rr)
    assert torch.equal(yt[-1], yt[0]) and torch.equal(yt[tiles // 2], yt[0])
    assert bool((yt == yt[0]).all())
    assert torch.equal(m.view(tiles, blk)[-1], m[:blk]) and torch.equal(v.view(tiles, blk)[-1], v[:blk])
    del yt, y
    dx, dg, db = K.ln_backward(x, dy, gd, m, v, rows, 1e-5)
    dx_r, dg_r, db_r = R.ln_backward(xb, dyb, g, m_r, v_r, blk, 1e-5)
    assert_close(to_np(dx[:blk]), dx_r, "f16", "grad", "first tile dx")
    dxt = dx.view(tiles, blk, Rr)
    assert bool((dxt == dxt[0]).all())
    assert_close(to_np(dg) / tiles, dg_r, "f16", "pgrad", "dgamma / tiles")
    assert_close(to_np(db) / tiles, db_r, "f16", "pgrad", "dbeta / tiles")


@pytest.mark.parametrize("layout", ["planes", "channel_last"])
def test_batch_normalization_just_below_2_31_elements(layout):
    _need(24)
    c, sp = 256, 4096
    n = ((1 << 31) - 1) // (c * sp)                  # 2047 samples -> 2 146 435 072 elements
    rng = np.random.default_rng(62)
    shape_b = (1, c, sp) if layout == "planes" else (1, sp, c)
    axis = 1 if layout == "planes" else 2
    xb = (rng.standard_normal(shape_b) * 2 + 1).astype(np.float16)
    dyb = rng.standard_normal(shape_b).astype(np.float16)
    g = rng.uniform(0.5, 1.5, c).astype(np.float32)
    b = (rng.standard_normal(c) * 0.1).astype(np.float32)
    x = torch.from_numpy(xb).cuda().repeat(n, 1, 1)
    dy = torch.from_numpy(dyb).cuda().repeat(n, 1, 1)
    assert x.numel() < (1 << 31) and x.numel() > (1 << 31) - (1 << 21)
    gd, bd = to_dev(g), to_dev(b)
    # statistics of n identical samples are those of one sample
    y_r, m_r, v_r, _, _ = R.bn_forward_batch(xb, b, g, None, None, axis, 0.9, 1e-5)
    y, m, v = K.bn_forward_batch(x, bd, gd, None, None, axis, 0.9, 1e-5)
    assert_close(to_np(m), m_r, "f16", "stat", "mean")
    assert_close(to_np(v), v_r, "f16", "stat", "var")
    assert_close(to_np(y[:1]), y_r, "f16", "y", "first sample y")
    assert bool((y == y[0]).all())
    del y
    # backward of the tiled batch: sums scale with n, dx = per-sample result with N -> n*N
    dx, dg, db = K.bn_backward(x, dy, gd, m, v, axis, 1e-5)
    dx_r, dg_r, db_r = R.bn_backward_batch(xb, dyb, g, m_r, v_r, axis, 1e-5)
    assert bool((dx == dx[0]).all())
    assert_close(to_np(dx[:1]), dx_r, "f16", "grad", "first sample dx")
    assert_close(to_np(dg) / n, dg_r, "f16", "pgrad", "dgamma / n")
    assert_close(to_np(db) / n, db_r, "f16", "pgrad", "dbeta / n")


@pytest.mark.parametrize("kind", ["gn", "in", "gn_cl", "in_cl"])
def test_group_and_instance_normalization_just_below_2_31_elements(kind):
    _need(24)
    c, sp, groups = 256, 4096, 32
    n = ((1 << 31) - 1) // (c * sp)
    cl = kind.endswith("_cl")
    rng = np.random.default_rng(63)
    shape_b = (1, sp, c) if cl else (1, c, sp)
    xb = (rng.standard_normal(shape_b) * 1.5).astype(np.float16)
    dyb = rng.standard_normal(shape_b).astype(np.float16)
    g = rng.uniform(0.5, 1.5, c).astype(np.float32)
    b = (rng.standard_normal(c) * 0.1).astype(np.float32)
    x = torch.from_numpy(xb).cuda().repeat(n, 1, 1)
    dy = torch.from_numpy(dyb).cuda().repeat(n, 1, 1)
    gd, bd = to_dev(g), to_dev(b)
    xt = np.moveaxis(xb, -1, 1) if cl else xb
    dyt = np.moveaxis(dyb, -1, 1) if cl else dyb
    back = (lambda a: np.moveaxis(np.asarray(a).reshape(xt.shape), 1, -1)) if cl else \
        (lambda a: np.asarray(a).reshape(xt.shape))
    if kind.startswith("gn"):
        y, m, v = K.gn_forward(x, bd, gd, groups, 1e-5, channel_last=cl)
        y_r, m_r, v_r = R.gn_forward(xt, b, g, 1, c, groups, 1e-5)
        dx_r, dg_r, db_r = R.gn_backward(xt, dyt, g, m_r, v_r, 1, c, groups, 1e-5)
    else:
        y, m, v = K.in_forward(x, bd, gd, 1e-5, channel_last=cl)
        y_r, m_r, v_r = R.in_forward(xt, b, g, 1, c, 1e-5)
        dx_r, dg_r, db_r = R.in_backward(xt, dyt, g, m_r, v_r, 1, c, 1e-5)
    per = m.numel() // n
    assert_close(to_np(m[:per]), m_r, "f16", "stat", "first sample mean")
    assert torch.equal(m.view(n, per)[-1], m[:per])
    assert_close(to_np(y[:1]), back(y_r), "f16", "y", "first sample y")
    assert bool((y == y[0]).all())
    del y
    if kind.startswith("gn"):
        dx, dg, db = K.gn_backward(x, dy, gd, m, v, groups, 1e-5, channel_last=cl)
    else:
        dx, dg, db = K.in_backward(x, dy, gd, m, v, 1e-5, channel_last=cl)
    assert_close(to_np(dx[:1]), back(dx_r), "f16", "grad", "first sample dx")
    assert bool((dx == dx[0]).all())
    assert_close(to_np(dg) / n, dg_r, "f16", "pgrad", "dgamma / n")
    assert_close(to_np(db) / n, db_r, "f16", "pgrad", "dbeta / n")


def test_one_unit_of_2_31_elements_is_refused():
    """Tensors of 2^31 elements and more run in ranges of rows / samples, but
    one row, one sample (for BatchNormalization: one slice of the axes ahead of
    the channel axis) must stay below 2^31 elements; the fused backward has no
    ranged form.  Refused before anything is launched (the buffers here hold
    16 elements)."""
    L = K.lib()
    s = torch.cuda.current_stream().cuda_stream
    t = torch.empty(16, device="cuda")
    p = t.data_ptr()
    assert L.nblahip_bn_fwd_infer(p, p, p, None, None, p, 2, 1 << 16, 1 << 15, 1e-5, 1,
                                  s) == -3                 # 2^31 elements per slice
    assert L.nblahip_bn_workspace_bytes(2, 1 << 16, 1 << 15, 1) == 0
    assert L.nblahip_fused_bn_bwd(p, p, p, None, p, p, None, None, p, None, None, None, 0, 0, 0, 0,
                                  1 << 11, 1 << 10, 1 << 10, 1e-5, 1, 1, p, 0, s) == -3
    assert L.nblahip_in_fwd(p, None, None, p, p, p, 2, 1 << 16, 1 << 15, 1, 1, 1e-5, 1,
                            s) == -3                       # 2^31 elements per sample
    assert L.nblahip_ln_fwd(p, None, None, p, p, p, 2, 1 << 31, 1e-5, 1, s) == -3
    assert L.nblahip_gn_cl_fwd(p, None, None, p, p, p, 2, 1 << 16, 1 << 15, 1, 1e-5, 1, p, 0,
                               s) == -3


# ---------------------------------------------------------------------------
# 2^31 elements and more (the reference indexes the row normalizations with
# Size_t: layer_normalization.cu:99, group_normalization.cu:57-62): the C-ABI
# runs ranges of rows / samples below 2^31 elements each, the parameter
# gradients of the later ranges accumulating onto the first.  The input is a
# small block tiled along the batch; first, middle and last tile are held to
# the float64 oracle of the block (the last range is shorter and may take
# another thread layout, so tiles are compared to the oracle, not bit for bit
# to each other), statistics likewise, dgamma / dbeta to tiles x the block's.
def _tiles_close(t, n_tiles, ref, dn, kind, what):
    for k in (0, n_tiles // 2, n_tiles - 2, n_tiles - 1):
        assert_close(to_np(t[k]), ref, dn, kind, f"{what}, tile {k}")


@pytest.mark.parametrize("accum", [False, True])
def test_layer_normalization_above_2_31_elements(accum):
    _need(30)
    Rr, blk = 8192, 64
    tiles = (1 << 31) // (Rr * blk) + 5                # 4101 tiles -> 2 150 105 088 elements
    rows = tiles * blk
    assert rows * Rr > (1 << 31)
    rng = np.random.default_rng(71)
    xb = (rng.standard_normal((blk, Rr)) + rng.uniform(-3, 3, (blk, 1))).astype(np.float16)
    dyb = rng.standard_normal((blk, Rr)).astype(np.float16)
    g = (rng.standard_normal(Rr) * 0.1 + 1).astype(np.float32)
    b = (rng.standard_normal(Rr) * 0.1).astype(np.float32)
    x = torch.from_numpy(xb).cuda().repeat(tiles, 1)
    dy = torch.from_numpy(dyb).cuda().repeat(tiles, 1)
    gd, bd = to_dev(g), to_dev(b)
    y, m, v = K.ln_forward(x, bd, gd, rows, 1e-5)
    y_r, m_r, v_r = R.ln_forward(xb, b, g, blk, 1e-5)
    _tiles_close(y.view(tiles, blk, Rr), tiles, y_r, "f16", "y", "y")
    _tiles_close(m.view(tiles, blk), tiles, m_r, "f16", "stat", "mean")
    _tiles_close(v.view(tiles, blk), tiles, v_r, "f16", "stat", "var")
    del y
    pre_g = torch.full((Rr,), 3.0, device="cuda")
    pre_b = torch.full((Rr,), -2.0, device="cuda")
    dx, dg, db = K.ln_backward(x, dy, gd, m, v, rows, 1e-5,
                               dgamma=pre_g.clone() if accum else None,
                               dbeta=pre_b.clone() if accum else None,
                               accum=(False, accum, accum))
    dx_r, dg_r, db_r = R.ln_backward(xb, dyb, g, m_r, v_r, blk, 1e-5)
    _tiles_close(dx.view(tiles, blk, Rr), tiles, dx_r, "f16", "grad", "dx")
    off_g, off_b = (3.0, -2.0) if accum else (0.0, 0.0)
    assert_close((to_np(dg) - off_g) / tiles, dg_r, "f16", "pgrad", "dgamma / tiles")
    assert_close((to_np(db) - off_b) / tiles, db_r, "f16", "pgrad", "dbeta / tiles")


@pytest.mark.parametrize("kind", ["gn", "in", "in_per_sample", "gn_cl", "in_cl"])
def test_group_and_instance_normalization_above_2_31_elements(kind):
    _need(30)
    c, sp, groups = 256, 4096, 32
    n = (1 << 31) // (c * sp) + 3                      # 2051 samples
    cl = kind.endswith("_cl")
    per_sample = kind == "in_per_sample"
    rng = np.random.default_rng(73)
    shape_b = (1, sp, c) if cl else (1, c, sp)
    xb = (rng.standard_normal(shape_b) * 1.5).astype(np.float16)
    dyb = rng.standard_normal(shape_b).astype(np.float16)
    g = rng.uniform(0.5, 1.5, c).astype(np.float32)
    b = (rng.standard_normal(c) * 0.1).astype(np.float32)
    x = torch.from_numpy(xb).cuda().repeat(n, 1, 1)
    dy = torch.from_numpy(dyb).cuda().repeat(n, 1, 1)
    assert x.numel() > (1 << 31)
    gd, bd = to_dev(g), to_dev(b)
    if per_sample:                                      # gamma / beta of shape [N, C]
        gd, bd = gd.repeat(n).contiguous(), bd.repeat(n).contiguous()
    xt = np.moveaxis(xb, -1, 1) if cl else xb
    dyt = np.moveaxis(dyb, -1, 1) if cl else dyb
    back = (lambda a: np.moveaxis(np.asarray(a).reshape(xt.shape), 1, -1)) if cl else \
        (lambda a: np.asarray(a).reshape(xt.shape))
    bc = not per_sample
    if kind.startswith("gn"):
        y, m, v = K.gn_forward(x, bd, gd, groups, 1e-5, channel_last=cl)
        y_r, m_r, v_r = R.gn_forward(xt, b, g, 1, c, groups, 1e-5)
        dx_r, dg_r, db_r = R.gn_backward(xt, dyt, g, m_r, v_r, 1, c, groups, 1e-5)
    else:
        y, m, v = K.in_forward(x, bd, gd, 1e-5, bc_gamma=bc, bc_beta=bc, channel_last=cl)
        y_r, m_r, v_r = R.in_forward(xt, b, g, 1, c, 1e-5)
        dx_r, dg_r, db_r = R.in_backward(xt, dyt, g, m_r, v_r, 1, c, 1e-5)
    per = m.numel() // n
    _tiles_close(m.view(n, per), n, np.asarray(m_r).ravel(), "f16", "stat", "mean")
    _tiles_close(v.view(n, per), n, np.asarray(v_r).ravel(), "f16", "stat", "var")
    _tiles_close(y, n, back(y_r)[0], "f16", "y", "y")
    del y
    if kind.startswith("gn"):
        dx, dg, db = K.gn_backward(x, dy, gd, m, v, groups, 1e-5, channel_last=cl)
    else:
        dx, dg, db = K.in_backward(x, dy, gd, m, v, 1e-5, bc_gamma=bc, bc_beta=bc, channel_last=cl)
    _tiles_close(dx, n, back(dx_r)[0], "f16", "grad", "dx")
    if per_sample:
        _tiles_close(dg.view(n, c), n, dg_r, "f16", "pgrad", "dgamma per sample")
        _tiles_close(db.view(n, c), n, db_r, "f16", "pgrad", "dbeta per sample")
    else:
        assert_close(to_np(dg) / n, dg_r, "f16", "pgrad", "dgamma / n")
        assert_close(to_np(db) / n, db_r, "f16", "pgrad", "dbeta / n")


@pytest.mark.parametrize("kind", ["gn_cl", "in_cl"])
def test_channel_last_batch_beyond_65535(kind):
    """70 000 samples: the channel-last kernels put the sample on a grid axis
    (65535 at most); the C-ABI runs them in two ranges.  The reference has no
    such limit (group_normalization.cu:57-62)."""
    n, blk, sp, c, groups = 70000, 8, (4, 4), 64, 8
    tiles = n // blk
    rng = np.random.default_rng(74)
    xb = (rng.standard_normal((blk,) + sp + (c,)) * 1.5 + rng.uniform(-1, 1, (blk, 1, 1, c))).astype(np.float16)
    dyb = rng.standard_normal((blk,) + sp + (c,)).astype(np.float16)
    g = rng.uniform(0.5, 1.5, c).astype(np.float32)
    b = (rng.standard_normal(c) * 0.1).astype(np.float32)
    x = torch.from_numpy(xb).cuda().repeat(tiles, 1, 1, 1)
    dy = torch.from_numpy(dyb).cuda().repeat(tiles, 1, 1, 1)
    gd, bd = to_dev(g), to_dev(b)
    xt, dyt = np.moveaxis(xb, -1, 1), np.moveaxis(dyb, -1, 1)
    back = lambda a: np.moveaxis(np.asarray(a).reshape(xt.shape), 1, -1)
    if kind == "gn_cl":
        y, m, v = K.gn_forward(x, bd, gd, groups, 1e-5, channel_last=True)
        dx, dg, db = K.gn_backward(x, dy, gd, m, v, groups, 1e-5, channel_last=True)
        y_r, m_r, v_r = R.gn_forward(xt, b, g, blk, c, groups, 1e-5)
        dx_r, dg_r, db_r = R.gn_backward(xt, dyt, g, m_r, v_r, blk, c, groups, 1e-5)
    else:
        y, m, v = K.in_forward(x, bd, gd, 1e-5, channel_last=True)
        dx, dg, db = K.in_backward(x, dy, gd, m, v, 1e-5, channel_last=True)
        y_r, m_r, v_r = R.in_forward(xt, b, g, blk, c, 1e-5)
        dx_r, dg_r, db_r = R.in_backward(xt, dyt, g, m_r, v_r, blk, c, 1e-5)
    per = m.numel() // tiles
    _tiles_close(m.view(tiles, per), tiles, np.asarray(m_r).ravel(), "f16", "stat", "mean")
    _tiles_close(y.view((tiles, blk) + sp + (c,)), tiles, back(y_r), "f16", "y", "y")
    _tiles_close(dx.view((tiles, blk) + sp + (c,)), tiles, back(dx_r), "f16", "grad", "dx")
    assert_close(to_np(dg) / tiles, dg_r, "f16", "pgrad", "dgamma / tiles")
    assert_close(to_np(db) / tiles, db_r, "f16", "pgrad", "dbeta / tiles")


@pytest.mark.parametrize("layout", ["planes", "channel_last"])
def test_batch_normalization_above_2_31_elements(layout):
    """A channel runs through the whole tensor, so the ranges are not
    independent: local statistics per range, their merge, normalization per
    range; backward: local sums per range, their sum, dx per range.  The batch
    is n1 copies of one sample followed by n2 copies of another, so that the
    two ranges (2047 + 4 samples) have different statistics and the merge must
    weight them; expected values from the two samples in float64."""
    _need(30)
    c, sp = 256, 4096
    n = (1 << 31) // (c * sp) + 3                      # 2051 samples, two ranges
    n2 = 100
    n1 = n - n2
    rng = np.random.default_rng(75)
    cl = layout == "channel_last"
    shape_b = (1, sp, c) if cl else (1, c, sp)
    axis = 2 if cl else 1
    xa = (rng.standard_normal(shape_b) * 2 + 1).astype(np.float16)
    xb = (rng.standard_normal(shape_b) * 0.5 - 2).astype(np.float16)
    dya = rng.standard_normal(shape_b).astype(np.float16)
    dyb = (rng.standard_normal(shape_b) * 2).astype(np.float16)
    g = rng.uniform(0.5, 1.5, c).astype(np.float32)
    b = (rng.standard_normal(c) * 0.1).astype(np.float32)
    x = torch.cat([torch.from_numpy(xa).cuda().repeat(n1, 1, 1), torch.from_numpy(xb).cuda().repeat(n2, 1, 1)])
    dy = torch.cat([torch.from_numpy(dya).cuda().repeat(n1, 1, 1), torch.from_numpy(dyb).cuda().repeat(n2, 1, 1)])
    assert x.numel() > (1 << 31) and x.is_contiguous()
    gd, bd = to_dev(g), to_dev(b)
    rm, rv = torch.zeros(c, device="cuda"), torch.ones(c, device="cuda")

    # float64 expectations per channel
    red = (0, 1) if cl else (0, 2)
    X = [xa.astype(np.float64), xb.astype(np.float64)]
    D = [dya.astype(np.float64), dyb.astype(np.float64)]
    W = [n1, n2]
    N = float(n) * sp
    mean = sum(w * a.sum(axis=red) for w, a in zip(W, X)) / N
    bshape = (1, 1, c) if cl else (1, c, 1)
    var = sum(w * ((a - mean.reshape(bshape)) ** 2).sum(axis=red) for w, a in zip(W, X)) / N
    istd = 1.0 / np.sqrt(var + 1e-5)
    G, Bt = g.astype(np.float64).reshape(bshape), b.astype(np.float64).reshape(bshape)
    XH = [(a - mean.reshape(bshape)) * istd.reshape(bshape) for a in X]
    Y = [xh * G + Bt for xh in XH]
    sdy = sum(w * d.sum(axis=red) for w, d in zip(W, D))
    sdx = sum(w * (d * xh).sum(axis=red) for w, d, xh in zip(W, D, XH))
    DX = [G * istd.reshape(bshape) * (d - sdy.reshape(bshape) / N - xh * sdx.reshape(bshape) / N)
          for d, xh in zip(D, XH)]

    y, m, v = K.bn_forward_batch(x, bd, gd, rm, rv, axis, 0.9, 1e-5)
    assert_close(to_np(m), mean, "f16", "stat", "mean")
    assert_close(to_np(v), var, "f16", "stat", "var")
    assert_close(to_np(rm), 0.1 * mean, "f16", "stat", "running mean")
    assert_close(to_np(rv), 0.9 + 0.1 * var * N / (N - 1), "f16", "stat", "running var")
    for k, which in ((0, 0), (n1 - 1, 0), (n1, 1), (n - 5, 1), (n - 1, 1)):
        assert_close(to_np(y[k:k + 1]), Y[which], "f16", "y", f"y of sample {k}")
    del y
    yi = K.bn_forward_global(x, bd, gd, m, v, axis, 1e-5)   # fixed statistics: elementwise ranges
    for k, which in ((0, 0), (n1, 1), (n - 1, 1)):
        assert_close(to_np(yi[k:k + 1]), Y[which], "f16", "y", f"inference y of sample {k}")
    del yi
    pre = torch.full((c,), 2.0, device="cuda")
    dx, dg, db = K.bn_backward(x, dy, gd, m, v, axis, 1e-5, dgamma=pre.clone(), dbeta=pre.clone(),
                               accum=(False, True, True))
    for k, which in ((0, 0), (n1 - 1, 0), (n1, 1), (n - 5, 1), (n - 1, 1)):
        assert_close(to_np(dx[k:k + 1]), DX[which], "f16", "grad", f"dx of sample {k}")
    assert_close((to_np(dg) - 2.0) / n, sdx / n, "f16", "pgrad", "dgamma / n")
    assert_close((to_np(db) - 2.0) / n, sdy / n, "f16", "pgrad", "dbeta / n")
