"""Pins for oracle/norm_ref.py: every oracle function is checked against
something that is NOT a retyping of its own formula - torch CPU float64
library routines with autograd, central finite differences, two-pass
statistics, brute-force enumeration and algebraic invariants."""
import itertools

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import norm_ref as R

RTOL = 1e-10
ATOL = 1e-10


def close(a, b, rtol=RTOL, atol=ATOL):
    np.testing.assert_allclose(np.asarray(a), np.asarray(b), rtol=rtol, atol=atol)


def T(a, grad=False):
    t = torch.tensor(np.asarray(a, dtype=np.float64), dtype=torch.float64)
    return t.requires_grad_(grad)


# ---------------------------------------------------------------- Welford
def test_welford_update_matches_two_pass():
    rng = np.random.default_rng(0)
    x = rng.standard_normal(37) * 3 + 5
    acc = R.welford_init()
    for v in x:
        acc = R.welford_update(acc, float(v))
    assert acc[2] == 37
    close(acc[0], x.mean())
    close(acc[1] / 37, x.var())


def test_welford_merge_every_split_tiny():
    rng = np.random.default_rng(1)
    for n in range(1, 9):
        x = rng.standard_normal(n) * 2 - 1
        for cut in range(0, n + 1):
            a = R.welford_init()
            for v in x[:cut]:
                a = R.welford_update(a, float(v))
            b = R.welford_init()
            for v in x[cut:]:
                b = R.welford_update(b, float(v))
            m = R.welford_merge(a, b)
            assert m[2] == n
            close(m[0], x.mean())
            close(m[1], ((x - x.mean()) ** 2).sum(), atol=1e-12)


def test_welford_merge_identity_and_associativity():
    rng = np.random.default_rng(2)
    parts = []
    for n in (3, 5, 2):
        acc = R.welford_init()
        for v in rng.standard_normal(n):
            acc = R.welford_update(acc, float(v))
        parts.append(acc)
    z = R.welford_init()
    assert R.welford_merge(z, parts[0]) == parts[0]
    assert R.welford_merge(parts[0], z) == parts[0]
    left = R.welford_merge(R.welford_merge(parts[0], parts[1]), parts[2])
    right = R.welford_merge(parts[0], R.welford_merge(parts[1], parts[2]))
    close(left[0], right[0])
    close(left[1], right[1])
    assert left[2] == right[2] == 10


def test_welford_rows_biased_variance():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, 23)) + np.arange(5)[:, None]
    m, v = R.welford_rows(x, chunk=7)
    close(m, x.mean(axis=1))
    close(v, x.var(axis=1))  # ddof=0 : m2 / R


# ---------------------------------------------------------------- BN
BN_CASES = [((4, 3, 5, 2), 1), ((6, 7), 1), ((3, 4, 5), 2), ((2, 3, 4, 5), 3),
            ((5, 1, 3), 1)]


@pytest.mark.parametrize("shape,axis", BN_CASES)
@pytest.mark.parametrize("no_scale,no_bias", [(False, False), (True, False),
                                              (False, True), (True, True)])
def test_bn_forward_global_vs_torch(shape, axis, no_scale, no_bias):
    rng = np.random.default_rng(10)
    c = shape[axis]
    x = rng.standard_normal(shape)
    g = None if no_scale else rng.uniform(0.5, 1.5, c)
    b = None if no_bias else rng.standard_normal(c)
    rm = rng.standard_normal(c) * 0.1
    rv = rng.uniform(0.5, 2, c)
    y = R.bn_forward_global(x, b, g, rm, rv, axis, 1e-5)
    xt = torch.movedim(T(x), axis, 1)
    yt = F.batch_norm(xt, T(rm), T(rv), None if g is None else T(g),
                      None if b is None else T(b), False, 0.1, 1e-5)
    close(y, torch.movedim(yt, 1, axis).numpy())


@pytest.mark.parametrize("splits", [[7], [3, 4], [1, 5, 2, 8], [10, 1]])
def test_syncbn_merge_equals_whole_batch_statistics(splits):
    """Per-shard (mean, biased var, count) folded by the reference's update
    equal the statistics of the concatenated batch; the running statistics
    equal torch's on the whole batch."""
    rng = np.random.default_rng(41)
    c = 5
    shards = [rng.standard_normal((n, c, 3, 2)) * (i + 1) + i for i, n in enumerate(splits)]
    means = np.stack([s.mean(axis=(0, 2, 3)) for s in shards])
    variances = np.stack([s.var(axis=(0, 2, 3)) for s in shards])
    counts = np.array([s.shape[0] * 6 for s in shards], np.float64)
    rm, rv = rng.standard_normal(c), rng.uniform(0.5, 2, c)
    mean, var, nrm, nrv = R.syncbn_merge_stats(means, variances, counts, rm, rv, 0.9)
    whole = np.concatenate(shards, axis=0)
    close(mean, whole.mean(axis=(0, 2, 3)))
    close(var, whole.var(axis=(0, 2, 3)))
    trm, trv = T(rm).clone(), T(rv).clone()
    F.batch_norm(T(whole), trm, trv, None, None, True, 0.1, 1e-5)
    close(nrm, trm.numpy())
    close(nrv, trv.numpy())


@pytest.mark.parametrize("shape,axis", BN_CASES)
@pytest.mark.parametrize("with_z", [True, False])
@pytest.mark.parametrize("batch_stat", [True, False])
def test_fused_bn_vs_torch_autograd(shape, axis, with_z, batch_stat):
    """relu(batch_norm(x) + z) and its gradients w.r.t. x, z, gamma, beta from
    torch float64 autograd, training and eval mode."""
    rng = np.random.default_rng(31)
    c = shape[axis]
    if batch_stat and int(np.prod(shape)) // c < 2:
        pytest.skip("degenerate")
    x = rng.standard_normal(shape) * 2 + 1
    z = rng.standard_normal(shape) if with_z else None
    dy = rng.standard_normal(shape)
    g = rng.uniform(0.5, 1.5, c)
    b = rng.standard_normal(c)
    rm = rng.standard_normal(c) * 0.3 + 1
    rv = rng.uniform(1.0, 4.0, c)
    y, mean, var, nrm, nrv = R.fused_bn_forward(x, z, b, g, rm, rv, axis, 0.9, 1e-5, batch_stat)
    xt, gt, bt = T(x, True), T(g, True), T(b, True)
    zt = T(z, True) if with_z else None
    trm, trv = T(rm).clone(), T(rv).clone()
    bn = F.batch_norm(torch.movedim(xt, axis, 1), trm, trv, gt, bt, batch_stat, 0.1, 1e-5)
    pre = torch.movedim(bn, 1, axis)
    if with_z:
        pre = pre + zt
    yt = torch.relu(pre)
    close(y, yt.detach().numpy())
    if c > 1:
        assert (y > 0).any() and (y == 0).any()  # both branches of the ReLU occur
    if batch_stat:
        close(nrm, trm.numpy())
        close(nrv, trv.numpy())
    (yt * T(dy)).sum().backward()
    st_m, st_v = (mean, var) if batch_stat else (rm, rv)
    dx, dz, dg, db = R.fused_bn_backward(x, y, dy, g, st_m, st_v, axis, 1e-5, batch_stat)
    close(dx, xt.grad.numpy(), rtol=1e-9, atol=1e-9)
    close(dg, gt.grad.numpy(), rtol=1e-9, atol=1e-9)
    close(db, bt.grad.numpy(), rtol=1e-9, atol=1e-9)
    if with_z:
        close(dz, zt.grad.numpy())
    # dz is dy gated by the sign of the OUTPUT (relu.cuh:59-61)
    np.testing.assert_array_equal(dz, np.where(y > 0, dy, 0.0))


@pytest.mark.parametrize("shape,axis", BN_CASES)
@pytest.mark.parametrize("decay", [0.9, 0.5])
def test_bn_forward_batch_vs_torch(shape, axis, decay):
    rng = np.random.default_rng(11)
    c = shape[axis]
    x = rng.standard_normal(shape) * 2 + 1
    g = rng.uniform(0.5, 1.5, c)
    b = rng.standard_normal(c)
    rm = rng.standard_normal(c)
    rv = rng.uniform(0.5, 2, c)
    y, mean, var, nrm, nrv = R.bn_forward_batch(x, b, g, rm, rv, axis, decay, 1e-5)
    xt = torch.movedim(T(x), axis, 1)
    trm, trv = T(rm).clone(), T(rv).clone()
    # NNabla decay_rate == 1 - torch momentum
    yt = F.batch_norm(xt, trm, trv, T(g), T(b), True, 1 - decay, 1e-5)
    close(y, torch.movedim(yt, 1, axis).numpy())
    close(nrm, trm.numpy())
    close(nrv, trv.numpy())           # unbiased N/(N-1) in the running var
    red = tuple(i for i in range(len(shape)) if i != axis)
    close(mean, x.mean(axis=red))
    close(var, x.var(axis=red))       # returned batch var is biased


def _torch_bn_train_with_stats(xt, g, b, eps):
    """BN built from primitive torch ops so that mean and var are graph
    nodes (needed to pin the 3-output dmean/dvar terms)."""
    red = [i for i in range(xt.dim()) if i != 1]
    mean = xt.mean(dim=red, keepdim=True)
    var = ((xt - mean) ** 2).mean(dim=red, keepdim=True)
    shape = [1, -1] + [1] * (xt.dim() - 2)
    y = (xt - mean) / torch.sqrt(var + eps)
    if g is not None:
        y = y * g.reshape(shape)
    if b is not None:
        y = y + b.reshape(shape)
    return y, mean.reshape(-1), var.reshape(-1)


@pytest.mark.parametrize("shape,axis", BN_CASES)
@pytest.mark.parametrize("no_scale", [False, True])
@pytest.mark.parametrize("with_stats_grad", [False, True])
def test_bn_backward_batch_vs_autograd(shape, axis, no_scale, with_stats_grad):
    rng = np.random.default_rng(12)
    c = shape[axis]
    if int(np.prod(shape)) // c < 2:
        pytest.skip("degenerate")
    x = rng.standard_normal(shape) * 2 + 1
    dy = rng.standard_normal(shape)
    g = None if no_scale else rng.uniform(0.5, 1.5, c)
    b = rng.standard_normal(c)
    dm = rng.standard_normal(c) if with_stats_grad else None
    dv = rng.standard_normal(c) if with_stats_grad else None
    _, mean, var, _, _ = R.bn_forward_batch(x, b, g, None, None, axis, 0.9, 1e-5)
    dx, dg, db = R.bn_backward_batch(x, dy, g, mean, var, axis, 1e-5, dm, dv)

    xt = T(x, True)
    gt = None if g is None else T(g, True)
    bt = T(b, True)
    xm = torch.movedim(xt, axis, 1)
    if with_stats_grad:
        yt, mt, vt = _torch_bn_train_with_stats(xm, gt, bt, 1e-5)
        loss = (yt * torch.movedim(T(dy), axis, 1)).sum() + (mt * T(dm)).sum() \
            + (vt * T(dv)).sum()
    else:
        yt = F.batch_norm(xm, None, None, gt, bt, True, 0.1, 1e-5)
        loss = (yt * torch.movedim(T(dy), axis, 1)).sum()
    loss.backward()
    close(dx, xt.grad.numpy(), rtol=1e-9, atol=1e-9)
    close(db, bt.grad.numpy())
    if gt is not None:
        close(dg, gt.grad.numpy(), rtol=1e-9, atol=1e-9)
    else:
        # dgamma is still defined (the gradient a unit gamma would receive)
        g1 = T(np.ones(c), True)
        y1 = F.batch_norm(torch.movedim(T(x), axis, 1), None, None, g1, T(b),
                          True, 0.1, 1e-5)
        (y1 * torch.movedim(T(dy), axis, 1)).sum().backward()
        close(dg, g1.grad.numpy(), rtol=1e-9, atol=1e-9)


@pytest.mark.parametrize("shape,axis", BN_CASES)
def test_bn_backward_global_vs_autograd(shape, axis):
    rng = np.random.default_rng(13)
    c = shape[axis]
    x = rng.standard_normal(shape)
    dy = rng.standard_normal(shape)
    g = rng.uniform(0.5, 1.5, c)
    b = rng.standard_normal(c)
    rm = rng.standard_normal(c) * 0.1
    rv = rng.uniform(0.5, 2, c)
    dx, dg, db = R.bn_backward_global(x, dy, g, rm, rv, axis, 1e-5)
    xt, gt, bt = T(x, True), T(g, True), T(b, True)
    yt = F.batch_norm(torch.movedim(xt, axis, 1), T(rm), T(rv), gt, bt, False,
                      0.1, 1e-5)
    (yt * torch.movedim(T(dy), axis, 1)).sum().backward()
    close(dx, xt.grad.numpy())
    close(dg, gt.grad.numpy())
    close(db, bt.grad.numpy())


def test_bn_backward_invariants():
    rng = np.random.default_rng(14)
    x = rng.standard_normal((6, 5, 7))
    dy = rng.standard_normal((6, 5, 7))
    g = rng.uniform(0.5, 1.5, 5)
    _, mean, var, _, _ = R.bn_forward_batch(x, None, g, None, None, 1, 0.9, 1e-5)
    dx, _, _ = R.bn_backward_batch(x, dy, g, mean, var, 1, 1e-5)
    close(dx.sum(axis=(0, 2)), np.zeros(5), atol=1e-12)
    xh = x - mean.reshape(1, 5, 1)
    # exact orthogonality holds for eps -> 0; with eps=1e-5 it is O(eps)
    close((dx * xh).sum(axis=(0, 2)), np.zeros(5), atol=1e-3)


def test_bn_constant_input_gives_beta():
    x = np.full((4, 3, 5), 2.5)
    b = np.array([0.1, -0.2, 0.3])
    y, mean, var, _, _ = R.bn_forward_batch(x, b, np.ones(3), None, None, 1, 0.9, 1e-5)
    close(var, np.zeros(3))
    close(y, np.broadcast_to(b.reshape(1, 3, 1), x.shape))


# ---------------------------------------------------------------- LN
LN_CASES = [((4, 6), 4), ((2, 3, 8), 6), ((2, 3, 8), 2), ((5, 1), 5), ((1, 17), 1)]


@pytest.mark.parametrize("shape,outer", LN_CASES)
@pytest.mark.parametrize("no_scale,no_bias", [(False, False), (True, True),
                                              (True, False), (False, True)])
def test_ln_forward_backward_vs_torch(shape, outer, no_scale, no_bias):
    rng = np.random.default_rng(20)
    x = rng.standard_normal(shape) + rng.uniform(-3, 3, (shape[0],) + (1,) * (len(shape) - 1))
    dy = rng.standard_normal(shape)
    Rr = int(np.prod(shape)) // outer
    nshape = None
    # normalized_shape = trailing dims whose product is R
    for k in range(len(shape) + 1):
        if int(np.prod(shape[k:])) == Rr:
            nshape = shape[k:]
            break
    g = None if no_scale else rng.standard_normal(Rr) * 0.1 + 1
    b = None if no_bias else rng.standard_normal(Rr) * 0.1
    y, mean, var = R.ln_forward(x, b, g, outer, 1e-5)
    dx, dg, db = R.ln_backward(x, dy, g, mean, var, outer, 1e-5)

    xt = T(x, True)
    gt = None if g is None else T(g.reshape(nshape), True)
    bt = None if b is None else T(b.reshape(nshape), True)
    yt = F.layer_norm(xt, nshape, gt, bt, 1e-5)
    (yt * T(dy)).sum().backward()
    close(y, yt.detach().numpy())
    close(dx, xt.grad.numpy(), rtol=1e-8, atol=1e-8)
    if gt is not None:
        close(dg, gt.grad.numpy().reshape(-1), rtol=1e-9, atol=1e-9)
    if bt is not None:
        close(db, bt.grad.numpy().reshape(-1))
    close(mean, x.reshape(outer, -1).mean(axis=1))
    close(var, x.reshape(outer, -1).var(axis=1))


def _torch_rows_with_stats(x2, eps):
    mean = x2.mean(dim=1, keepdim=True)
    var = ((x2 - mean) ** 2).mean(dim=1, keepdim=True)
    return (x2 - mean) / torch.sqrt(var + eps), mean.reshape(-1), var.reshape(-1)


def test_ln_backward_with_stat_grads_vs_autograd():
    rng = np.random.default_rng(21)
    outer, Rr = 5, 9
    x = rng.standard_normal((outer, Rr)) * 2 + 1
    dy = rng.standard_normal((outer, Rr))
    g = rng.standard_normal(Rr) * 0.1 + 1
    dm = rng.standard_normal(outer)
    dv = rng.standard_normal(outer)
    _, mean, var = R.ln_forward(x, None, g, outer, 1e-5)
    dx, dg, db = R.ln_backward(x, dy, g, mean, var, outer, 1e-5, dm, dv)
    xt, gt = T(x, True), T(g, True)
    xh, mt, vt = _torch_rows_with_stats(xt, 1e-5)
    ((xh * gt * T(dy)).sum() + (mt * T(dm)).sum() + (vt * T(dv)).sum()).backward()
    close(dx, xt.grad.numpy(), rtol=1e-9, atol=1e-9)
    close(dg, gt.grad.numpy(), rtol=1e-9, atol=1e-9)


def test_ln_backward_finite_difference():
    rng = np.random.default_rng(22)
    outer, Rr = 3, 6
    x = rng.standard_normal((outer, Rr))
    dy = rng.standard_normal((outer, Rr))
    g = rng.uniform(0.5, 1.5, Rr)
    b = rng.standard_normal(Rr)
    dm, dv = rng.standard_normal(outer), rng.standard_normal(outer)

    def loss(xv):
        y, m, v = R.ln_forward(xv, b, g, outer, 1e-5)
        return (y * dy).sum() + (m * dm).sum() + (v * dv).sum()

    _, mean, var = R.ln_forward(x, b, g, outer, 1e-5)
    dx, _, _ = R.ln_backward(x, dy, g, mean, var, outer, 1e-5, dm, dv)
    h = 1e-6
    num = np.zeros_like(x)
    for i, j in itertools.product(range(outer), range(Rr)):
        xp, xm = x.copy(), x.copy()
        xp[i, j] += h
        xm[i, j] -= h
        num[i, j] = (loss(xp) - loss(xm)) / (2 * h)
    close(dx, num, rtol=1e-6, atol=1e-7)


# ---------------------------------------------------------------- GN
GN_CASES = [(2, 8, (3, 3), 4), (3, 6, (5,), 2), (1, 4, (2, 2), 1), (2, 6, (4,), 6),
            (2, 4, (), 2)]


@pytest.mark.parametrize("n,c,sp,groups", GN_CASES)
@pytest.mark.parametrize("no_scale,no_bias", [(False, False), (True, True)])
def test_gn_forward_backward_vs_torch(n, c, sp, groups, no_scale, no_bias):
    rng = np.random.default_rng(30)
    shape = (n, c) + sp
    x = rng.standard_normal(shape) * 1.5
    dy = rng.standard_normal(shape)
    g = None if no_scale else rng.uniform(0.5, 1.5, c)
    b = None if no_bias else rng.standard_normal(c)
    y, mean, var = R.gn_forward(x, b, g, n, c, groups, 1e-5)
    dx, dg, db = R.gn_backward(x, dy, g, mean, var, n, c, groups, 1e-5)
    xt = T(x, True)
    gt = None if g is None else T(g, True)
    bt = None if b is None else T(b, True)
    yt = F.group_norm(xt, groups, gt, bt, 1e-5)
    (yt * T(dy)).sum().backward()
    close(y, yt.detach().numpy(), rtol=1e-9, atol=1e-9)
    close(dx, xt.grad.numpy(), rtol=1e-8, atol=1e-8)
    if gt is not None:
        close(dg, gt.grad.numpy(), rtol=1e-9, atol=1e-9)
    if bt is not None:
        close(db, bt.grad.numpy())
    close(mean, x.reshape(n * groups, -1).mean(axis=1))
    close(var, x.reshape(n * groups, -1).var(axis=1))


def test_gn_backward_with_stat_grads_vs_autograd():
    rng = np.random.default_rng(31)
    n, c, groups, sp = 2, 6, 3, 5
    x = rng.standard_normal((n, c, sp))
    dy = rng.standard_normal((n, c, sp))
    g = rng.uniform(0.5, 1.5, c)
    dm = rng.standard_normal(n * groups)
    dv = rng.standard_normal(n * groups)
    _, mean, var = R.gn_forward(x, None, g, n, c, groups, 1e-5)
    dx, dg, _ = R.gn_backward(x, dy, g, mean, var, n, c, groups, 1e-5, dm, dv)
    xt, gt = T(x, True), T(g, True)
    xh, mt, vt = _torch_rows_with_stats(xt.reshape(n * groups, -1), 1e-5)
    yt = xh.reshape(n, c, sp) * gt.reshape(1, c, 1)
    ((yt * T(dy)).sum() + (mt * T(dm)).sum() + (vt * T(dv)).sum()).backward()
    close(dx, xt.grad.numpy(), rtol=1e-9, atol=1e-9)
    close(dg, gt.grad.numpy(), rtol=1e-9, atol=1e-9)


# ---------------------------------------------------------------- IN
@pytest.mark.parametrize("n,c,sp", [(2, 3, (4, 4)), (3, 5, (7,)), (1, 2, (3, 2))])
@pytest.mark.parametrize("affine", [True, False])
def test_in_forward_backward_vs_torch(n, c, sp, affine):
    rng = np.random.default_rng(40)
    shape = (n, c) + sp
    x = rng.standard_normal(shape) * 1.5
    dy = rng.standard_normal(shape)
    g = rng.uniform(0.5, 1.5, c) if affine else None
    b = rng.standard_normal(c) if affine else None
    y, mean, var = R.in_forward(x, b, g, n, c, 1e-5)
    dx, dg, db = R.in_backward(x, dy, g, mean, var, n, c, 1e-5)
    xt = T(x, True)
    gt = T(g, True) if affine else None
    bt = T(b, True) if affine else None
    yt = F.instance_norm(xt, None, None, gt, bt, True, 0.1, 1e-5)
    (yt * T(dy)).sum().backward()
    close(y, yt.detach().numpy(), rtol=1e-9, atol=1e-9)
    close(dx, xt.grad.numpy(), rtol=1e-8, atol=1e-8)
    if affine:
        close(dg, gt.grad.numpy(), rtol=1e-9, atol=1e-9)
        close(db, bt.grad.numpy())


def test_in_per_sample_affine_vs_autograd():
    """gamma/beta of shape [N, C] (no broadcast over the batch) with
    dmean/dvar flowing back."""
    rng = np.random.default_rng(41)
    n, c, sp = 3, 4, 6
    x = rng.standard_normal((n, c, sp))
    dy = rng.standard_normal((n, c, sp))
    g = rng.uniform(0.5, 1.5, n * c)
    b = rng.standard_normal(n * c)
    dm, dv = rng.standard_normal(n * c), rng.standard_normal(n * c)
    y, mean, var = R.in_forward(x, b, g, n, c, 1e-5)
    dx, dg, db = R.in_backward(x, dy, g, mean, var, n, c, 1e-5, dm, dv,
                               bc_gamma=False, bc_beta=False)
    xt, gt, bt = T(x, True), T(g, True), T(b, True)
    xh, mt, vt = _torch_rows_with_stats(xt.reshape(n * c, -1), 1e-5)
    yt = xh * gt[:, None] + bt[:, None]
    ((yt * T(dy).reshape(n * c, -1)).sum() + (mt * T(dm)).sum()
     + (vt * T(dv)).sum()).backward()
    close(y, yt.detach().numpy().reshape(n, c, sp))
    close(dx, xt.grad.numpy(), rtol=1e-9, atol=1e-9)
    close(dg, gt.grad.numpy(), rtol=1e-9, atol=1e-9)
    close(db, bt.grad.numpy())


def test_gn_with_one_channel_per_group_equals_in():
    rng = np.random.default_rng(42)
    n, c, sp = 2, 4, 9
    x = rng.standard_normal((n, c, sp))
    g = rng.uniform(0.5, 1.5, c)
    b = rng.standard_normal(c)
    y1, m1, v1 = R.gn_forward(x, b, g, n, c, c, 1e-5)
    y2, m2, v2 = R.in_forward(x, b, g, n, c, 1e-5)
    close(y1, y2)
    close(m1, m2)
    close(v1, v2)
