#!/usr/bin/env python3
"""Writes the golden vectors of tests/golden/*.npz.

The reference tree holds no stored vectors for the normalization functions and
cannot be built or run in this image, so the expected outputs come from an
implementation that shares no code with this repository's oracle or kernels:
PyTorch's CPU operators in float64 (F.batch_norm / layer_norm / group_norm /
instance_norm) with autograd for every gradient, including the gradients that
flow in through the mean and variance outputs.  Shapes are small versions of
the benchmark configurations with their input distributions.

Each file holds the inputs (already rounded to the storage dtype named in
`dtype`, stored as float32) and the expected outputs as float64 arrays.  Run from the repository
root:  python tests/golden/make_fixtures.py
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
EPS = 1e-5
DECAY = 0.9


def rounded(a, dtype):
    """float64 array holding values exactly representable in `dtype`."""
    t = torch.from_numpy(np.asarray(a, np.float64))
    return t.to(torch.float16 if dtype == "f16" else torch.float32).to(torch.float64).numpy()


def t64(a, grad=False):
    t = torch.from_numpy(np.asarray(a, np.float64)).clone()
    return t.requires_grad_(grad)


INPUTS = ("x", "dy", "gamma", "beta", "rmean", "rvar", "dmean", "dvar")


def save(name, **arrays):
    # inputs are float32-representable by construction: store them as float32
    for k in INPUTS:
        if k in arrays:
            assert np.array_equal(arrays[k].astype(np.float32).astype(np.float64), arrays[k])
            arrays[k] = arrays[k].astype(np.float32)
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)
    print("wrote", name, {k: getattr(v, "shape", None) for k, v in arrays.items()})


def bn_case(name, shape, axis, dtype, seed, mean=0.0, std=1.0, outliers=False, stat_grads=False):
    rng = np.random.default_rng(seed)
    c = shape[axis]
    x = rng.standard_normal(shape) * std + mean
    if outliers:
        x = np.where(rng.random(shape) < 0.01, x * 50, x)
    x = rounded(x, dtype)
    dy = rounded(rng.standard_normal(shape), dtype)
    gamma = rounded(rng.uniform(0.5, 1.5, c), "f32")
    beta = rounded(rng.standard_normal(c) * 0.1, "f32")
    rmean = rounded(rng.standard_normal(c) * 0.1, "f32")
    rvar = rounded(rng.uniform(0.5, 2.0, c), "f32")
    dmean = rounded(rng.standard_normal(c), "f32")
    dvar = rounded(rng.standard_normal(c), "f32")

    # torch wants the channel at axis 1
    xt = t64(np.moveaxis(x, axis, 1), grad=True)
    dyt = t64(np.moveaxis(dy, axis, 1))
    g, b = t64(gamma, True), t64(beta, True)
    rm, rv = t64(rmean), t64(rvar)
    y = F.batch_norm(xt, rm, rv, g, b, training=True, momentum=1.0 - DECAY, eps=EPS)
    red = [d for d in range(xt.dim()) if d != 1]
    bmean = xt.mean(dim=red)
    bvar = xt.var(dim=red, unbiased=False)
    loss = (y * dyt).sum()
    if stat_grads:
        loss = loss + (bmean * t64(dmean)).sum() + (bvar * t64(dvar)).sum()
    dx, dg, db = torch.autograd.grad(loss, [xt, g, b])
    # inference mode on the same tensor with the original running statistics
    yi = F.batch_norm(t64(np.moveaxis(x, axis, 1)), t64(rmean), t64(rvar), t64(gamma), t64(beta),
                      training=False, eps=EPS)
    back = lambda t: np.ascontiguousarray(np.moveaxis(t.detach().numpy(), 1, axis))
    save(name, kind="bn", dtype=dtype, axis=axis, eps=EPS, decay_rate=DECAY,
         stat_grads=int(stat_grads), x=x, dy=dy, gamma=gamma, beta=beta, rmean=rmean, rvar=rvar,
         dmean=dmean, dvar=dvar, y=back(y), mean=bmean.detach().numpy(),
         var=bvar.detach().numpy(), rmean_out=rm.numpy(), rvar_out=rv.numpy(), dx=back(dx),
         dgamma=dg.numpy(), dbeta=db.numpy(), y_inference=back(yi))


def ln_case(name, outer, R, dtype, seed, stat_grads=False):
    rng = np.random.default_rng(seed)
    x = rounded(rng.standard_normal((outer, R)) + rng.uniform(-3, 3, (outer, 1)), dtype)
    dy = rounded(rng.standard_normal((outer, R)), dtype)
    gamma = rounded(rng.standard_normal(R) * 0.1 + 1, "f32")
    beta = rounded(rng.standard_normal(R) * 0.1, "f32")
    dmean = rounded(rng.standard_normal(outer), "f32")
    dvar = rounded(rng.standard_normal(outer), "f32")
    xt, g, b = t64(x, True), t64(gamma, True), t64(beta, True)
    y = F.layer_norm(xt, (R,), g, b, EPS)
    m, v = xt.mean(dim=1), xt.var(dim=1, unbiased=False)
    loss = (y * t64(dy)).sum()
    if stat_grads:
        loss = loss + (m * t64(dmean)).sum() + (v * t64(dvar)).sum()
    dx, dg, db = torch.autograd.grad(loss, [xt, g, b])
    save(name, kind="ln", dtype=dtype, eps=EPS, stat_grads=int(stat_grads), x=x, dy=dy,
         gamma=gamma, beta=beta, dmean=dmean, dvar=dvar, y=y.detach().numpy(),
         mean=m.detach().numpy(), var=v.detach().numpy(), dx=dx.numpy(), dgamma=dg.numpy(),
         dbeta=db.numpy())


def gn_case(name, n, c, sp, groups, dtype, seed, stat_grads=False):
    """groups == c is InstanceNormalization (F.instance_norm is used then)."""
    rng = np.random.default_rng(seed)
    shape = (n, c) + sp
    x = rounded(rng.standard_normal(shape) * 1.5, dtype)
    dy = rounded(rng.standard_normal(shape), dtype)
    gamma = rounded(rng.uniform(0.5, 1.5, c), "f32")
    beta = rounded(rng.standard_normal(c) * 0.1, "f32")
    dmean = rounded(rng.standard_normal(n * groups), "f32")
    dvar = rounded(rng.standard_normal(n * groups), "f32")
    xt, g, b = t64(x, True), t64(gamma, True), t64(beta, True)
    if groups == c:
        y = F.instance_norm(xt, weight=g, bias=b, use_input_stats=True, eps=EPS)
    else:
        y = F.group_norm(xt, groups, g, b, EPS)
    xg = xt.reshape(n * groups, -1)
    m, v = xg.mean(dim=1), xg.var(dim=1, unbiased=False)
    loss = (y * t64(dy)).sum()
    if stat_grads:
        loss = loss + (m * t64(dmean)).sum() + (v * t64(dvar)).sum()
    dx, dg, db = torch.autograd.grad(loss, [xt, g, b])
    save(name, kind="gn", dtype=dtype, eps=EPS, groups=groups, stat_grads=int(stat_grads), x=x,
         dy=dy, gamma=gamma, beta=beta, dmean=dmean, dvar=dvar, y=y.detach().numpy(),
         mean=m.detach().numpy(), var=v.detach().numpy(), dx=dx.numpy(), dgamma=dg.numpy(),
         dbeta=db.numpy())


def main():
    # benchmark configuration 1/2: BatchNormalization NCHW fp32, x ~ N(1,2)
    bn_case("bn_nchw_f32", (4, 16, 7, 7), 1, "f32", 1, mean=1.0, std=2.0)
    bn_case("bn_nchw_f32_stat_grads", (5, 12, 6, 5), 1, "f32", 11, mean=1.0, std=2.0,
            stat_grads=True)
    bn_case("bn_nchw_f16_planes_in_registers", (8, 24, 4, 4), 1, "f16", 12)
    # configuration 5: channel-last fp16 with 1 % outliers x50
    bn_case("bn_nhwc_f16_outliers", (4, 6, 5, 32), 3, "f16", 4, outliers=True)
    bn_case("bn_nhwc_f32", (20, 3, 2, 24), 3, "f32", 14)
    bn_case("bn_2d_f32", (37, 20), 1, "f32", 15)
    # configuration 3: LayerNormalization, rows with offsets, fp32 and fp16
    ln_case("ln_f32", 24, 96, "f32", 2)
    ln_case("ln_f16", 24, 96, "f16", 2)
    ln_case("ln_f32_long_rows_stat_grads", 2, 2500, "f32", 22, stat_grads=True)
    # configuration 4: GroupNormalization fp16 and InstanceNormalization on the same tensor
    gn_case("gn_f16", 3, 16, (6, 6), 4, "f16", 3)
    gn_case("in_f16", 3, 16, (6, 6), 16, "f16", 3)
    gn_case("gn_f32_stat_grads", 2, 12, (5, 7), 3, "f32", 33, stat_grads=True)
    gn_case("in_f32_stat_grads", 2, 12, (5, 7), 12, "f32", 34, stat_grads=True)
    gn_case("gn_f32_one_group", 2, 6, (9,), 1, "f32", 35)
    # shapes of the plans that came later: planes that are no whole number of
    # 16-byte vectors (7x7: channel packs / rows; 17x17: masked vectors), an odd
    # hidden size, odd planes for Instance / GroupNormalization, and a tensor
    # wide enough for the channel-last kernels (tests run it channel-last too)
    bn_case("bn_nchw_f16_7x7_planes", (8, 24, 7, 7), 1, "f16", 41)
    bn_case("bn_nchw_f32_17x17_planes", (5, 4, 17, 17), 1, "f32", 42, mean=1.0, std=2.0)
    ln_case("ln_f16_odd_hidden", 5, 1023, "f16", 43)
    ln_case("ln_f32_odd_hidden_stat_grads", 4, 515, "f32", 44, stat_grads=True)
    gn_case("in_f16_odd_planes", 2, 6, (15, 15), 6, "f16", 45)
    gn_case("gn_f16_odd_planes", 2, 8, (9, 7), 2, "f16", 46)
    gn_case("gn_f16_wide", 2, 64, (8, 8), 8, "f16", 47)
    gn_case("in_f16_wide", 2, 64, (8, 8), 64, "f16", 48)


if __name__ == "__main__":
    main()
