"""BatchNormalization of a batch split over several workers (the device steps
of SyncBatchNormalization, sync_batch_normalization.cu:86-285) on ONE GPU: the
shards are processed one after the other, the all-gather / all-reduce between
the steps is a concatenation / a sum on the device, and the result must equal
the oracle's BatchNormalization of the whole batch."""
import numpy as np
import pytest
import torch

from _util import assert_close, dtype_name, load_package, rounded, to_dev, to_np
from oracle import norm_ref as R

pytestmark = pytest.mark.gpu
K = load_package()
DTYPES = [torch.float32, torch.float16]

# (per-worker batch sizes, rest of the shape, channel axis)
CASES = [
    ([4], (8, 6, 6), 1),                 # one worker: plain BatchNormalization
    ([2, 2], (8, 6, 6), 1),
    ([1, 3, 2], (5, 7, 3), 1),           # uneven shards, odd sizes
    ([3, 5], (4, 4, 16), 3),             # channel-last
    ([2, 1, 1, 4], (7, 7, 24), 3),       # channel-last, generic apply
    ([8, 8], (256, 9, 9), 1),            # channel-owning reduction blocks
    ([5, 9], (24,), 1),                  # 2-D input
]


def make(splits, rest, axis, dtype, seed):
    rng = np.random.default_rng(seed)
    n = sum(splits)
    shape = (n,) + rest
    c = shape[axis]
    x = rounded(rng.standard_normal(shape) * 2.0 + np.arange(n).reshape((n,) + (1,) * len(rest)) * 0.1,
                dtype)
    dy = rounded(rng.standard_normal(shape), dtype)
    g = rng.uniform(0.5, 1.5, c).astype(np.float32).astype(np.float64)
    b = (rng.standard_normal(c) * 0.1).astype(np.float32).astype(np.float64)
    rm = (rng.standard_normal(c) * 0.1).astype(np.float32).astype(np.float64)
    rv = rng.uniform(0.5, 2.0, c).astype(np.float32).astype(np.float64)
    return x, dy, g, b, rm, rv


@pytest.mark.parametrize("splits,rest,axis", CASES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_split_batch_equals_whole_batch(splits, rest, axis, dtype):
    dn = dtype_name(dtype)
    x, dy, g, b, rm, rv = make(splits, rest, axis, dtype, 51)
    c = x.shape[axis]
    per_sample = int(np.prod(x.shape)) // (x.shape[0] * c)
    y_r, m_r, v_r, rm_r, rv_r = R.bn_forward_batch(x, b, g, rm, rv, axis, 0.9, 1e-5)
    dx_r, dg_r, db_r = R.bn_backward_batch(x, dy, g, m_r, v_r, axis, 1e-5)

    bounds = np.cumsum([0] + list(splits))
    xs = [to_dev(np.ascontiguousarray(x[a:e]), dtype) for a, e in zip(bounds[:-1], bounds[1:])]
    dys = [to_dev(np.ascontiguousarray(dy[a:e]), dtype) for a, e in zip(bounds[:-1], bounds[1:])]
    gd, bd, rmd, rvd = to_dev(g), to_dev(b), to_dev(rm), to_dev(rv)

    # forward: local statistics, "all-gather", merge, apply
    records = []
    for xi, n_i in zip(xs, splits):
        m_i, v_i = K.bn_local_stats(xi, axis)
        cnt = torch.tensor([float(n_i * per_sample)], device="cuda")
        records.append(torch.cat([m_i, v_i, cnt]))
    stats = torch.stack(records).contiguous()
    mean, var = K.bn_merge_stats(stats, c, rmd, rvd, 0.9)
    assert_close(to_np(mean), m_r, dn, "stat", "mean")
    assert_close(to_np(var), v_r, dn, "stat", "var")
    assert_close(to_np(rmd), rm_r, dn, "stat", "running_mean")
    assert_close(to_np(rvd), rv_r, dn, "stat", "running_var")
    ys = [K.bn_forward_global(xi, bd, gd, mean, var, axis, 1e-5) for xi in xs]
    assert_close(np.concatenate([to_np(t) for t in ys]), y_r, dn, "y", "y")

    # backward: local pairs, "all-reduce", apply; dgamma/dbeta add up over workers
    sums = torch.zeros(c, 2, device="cuda")
    dg = torch.zeros(c, device="cuda")
    db = torch.zeros(c, device="cuda")
    for xi, dyi in zip(xs, dys):
        s_i, dg_i, db_i = K.bn_backward_local_sums(xi, dyi, mean, var, axis, 1e-5)
        sums += s_i
        dg += dg_i
        db += db_i
    total = float(sum(splits) * per_sample)
    dxs = [K.bn_backward_apply_sums(xi, dyi, gd, mean, var, sums, total, axis, 1e-5)
           for xi, dyi in zip(xs, dys)]
    assert_close(np.concatenate([to_np(t) for t in dxs]), dx_r, dn, "grad", "dx")
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


def test_one_worker_is_bitwise_the_plain_path():
    """(With the plain path on the same split reduction: the kernels that hold
    a channel on one CU or split it over several blocks, which take this shape
    by default, and the single-pass row kernels sum in another order and are
    switched off for the comparison.)"""
    torch.manual_seed(3)
    x = torch.randn(64, 8, 48, 48, device="cuda")
    dy = torch.randn_like(x)
    g = torch.rand(8, device="cuda") + 0.5
    b = torch.randn(8, device="cuda")
    K.tune_reset()
    K.tune_set("BN_CHAN_SPLIT", 0)
    K.tune_set("BN_ONCHIP", 0)
    try:
        y0, m0, v0 = K.bn_forward_batch(x, b, g, None, None, 1, 0.9, 1e-5)
        dx0, dg0, db0 = K.bn_backward(x, dy, g, m0, v0, 1, 1e-5)
        m, v = K.bn_local_stats(x, 1)
        sums, dg, db = K.bn_backward_local_sums(x, dy, m, v, 1, 1e-5)
        dx = K.bn_backward_apply_sums(x, dy, g, m, v, sums, 64 * 48 * 48, 1, 1e-5)
    finally:
        K.tune_reset()
    assert torch.equal(m, m0) and torch.equal(v, v0)
    assert torch.equal(dg, dg0) and torch.equal(db, db0)
    assert torch.equal(dx, dx0)


def test_three_output_terms_and_accumulation():
    """dmean/dvar of the three-output form enter the apply step; accum adds."""
    splits, rest, axis = [2, 3], (6, 5, 5), 1
    x, dy, g, b, rm, rv = make(splits, rest, axis, torch.float32, 52)
    c = 6
    rng = np.random.default_rng(53)
    dm, dv = rng.standard_normal(c), rng.standard_normal(c)
    _, m_r, v_r, _, _ = R.bn_forward_batch(x, b, g, None, None, axis, 0.9, 1e-5)
    dx_r, _, _ = R.bn_backward_batch(x, dy, g, m_r, v_r, axis, 1e-5, dm, dv)
    xs = [to_dev(np.ascontiguousarray(x[:2])), to_dev(np.ascontiguousarray(x[2:]))]
    dys = [to_dev(np.ascontiguousarray(dy[:2])), to_dev(np.ascontiguousarray(dy[2:]))]
    mean, var = to_dev(m_r), to_dev(v_r)
    sums = sum(K.bn_backward_local_sums(xi, dyi, mean, var, axis, 1e-5, need_params=False)[0]
               for xi, dyi in zip(xs, dys))
    pre = rng.standard_normal(x.shape).astype(np.float32)
    outs = []
    for xi, dyi, pi in zip(xs, dys, (pre[:2], pre[2:])):
        dxd = to_dev(np.ascontiguousarray(pi))
        K.bn_backward_apply_sums(xi, dyi, to_dev(g), mean, var, sums.contiguous(), 5 * 25, axis, 1e-5,
                                 dmean=to_dev(dm), dvar=to_dev(dv), dx=dxd, accum=True)
        outs.append(to_np(dxd))
    assert_close(np.concatenate(outs), dx_r + pre, "f32", "grad", "dx accum with dmean/dvar")


def test_split_batch_argument_errors():
    L = K.lib()
    s = torch.cuda.current_stream().cuda_stream
    x = torch.randn(4, 8, 16, device="cuda")
    m = torch.zeros(8, device="cuda")
    ws = torch.empty(max(1, L.nblahip_bn_workspace_bytes(4, 8, 16, 0)), dtype=torch.uint8,
                     device="cuda")
    assert L.nblahip_bn_local_stats(x.data_ptr(), None, m.data_ptr(), 4, 8, 16, 0, ws.data_ptr(),
                                    ws.numel(), s) == -1
    assert L.nblahip_bn_local_stats(x.data_ptr(), m.data_ptr(), m.data_ptr(), 4, 8, 16, 0, None, 0,
                                    s) == -2
    assert L.nblahip_bn_merge_stats(None, 2, 8, m.data_ptr(), m.data_ptr(), None, None, 0.9,
                                    s) == -1
    assert L.nblahip_bn_merge_stats(None, 0, 8, None, None, None, None, 0.9, s) == 0
    sums = torch.zeros(8, 2, device="cuda")
    assert L.nblahip_bn_bwd_apply_sums(x.data_ptr(), x.data_ptr(), None, m.data_ptr(), m.data_ptr(),
                                       sums.data_ptr(), 0.0, None, None, x.data_ptr(), 0, 4, 8, 16,
                                       1e-5, 0, ws.data_ptr(), ws.numel(), s) == -1   # count < 1
