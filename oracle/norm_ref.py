"""CPU oracle for the normalization-reduction path (TEST INFRASTRUCTURE ONLY).

This module restates, in NumPy float64, the arithmetic that sony/nnabla-ext-cuda
performs for BatchNormalization, LayerNormalization, GroupNormalization and
InstanceNormalization.  It exists to CHECK the HIP kernels: only tests, the smoke
check and the CPU-baseline leg of the benchmark may import it.  The product
path never does.

Canonical layouts (row-major, the reference's own flattening):
  BN      x viewed as [size0, C, size2]   (batch_normalization.cu:34-35,195-198)
  LN      x viewed as [outer, R]          (layer_normalization.cu:53-59)
  GN/IN   x viewed as [N, C, spatial]     (group_normalization.cu:57-62,
                                           instance_normalization.cu:53-55)

How each function is pinned (see tests/test_oracle_pins.py; the same torch
operators also wrote the stored vectors of tests/golden/*.npz, which
tests/test_golden.py holds the oracle and the HIP path to):
  bn_forward_global, bn_forward_batch, bn_backward_batch, bn_backward_global,
  ln_forward/backward, gn_forward/backward, in_forward/backward
      -> torch CPU float64 F.batch_norm / layer_norm / group_norm /
         instance_norm + autograd (library routines), incl. the 3-output
         dmean/dvar terms through an autograd loss that consumes mean and var;
  syncbn_merge_stats
      -> equality with the statistics of the concatenated batch (two-pass
         numpy mean/var) for even and uneven splits, and with torch's running
         statistics of the whole batch;
  fused_bn_forward / fused_bn_backward
      -> torch CPU float64 relu(F.batch_norm(x) + z) + autograd (training and
         eval mode, with and without z);
  welford_update / welford_merge / welford_rows
      -> equality with the two-pass mean/variance, merge associativity,
         brute-force split enumeration on tiny inputs, n=0 identity;
  all backward functions
      -> central finite differences in float64 and the sum(dx)=0,
         sum(dx*xhat)=0 invariants.
Conventions only the absent NNabla core could pin (inference-mode backward,
stat output shapes, the gamma/beta broadcast rule of InstanceNormalization)
follow the textbook definition and are "convention unpinned".

All citations are file:line under the reference tree.
"""
from __future__ import annotations

import numpy as np

F64 = np.float64


def _f64(a):
    return None if a is None else np.asarray(a, dtype=F64)


# --------------------------------------------------------------------------
# Welford (include/nbla/cuda/utils/reduce_ops/welford.cuh:62-103)
# --------------------------------------------------------------------------
def welford_init():
    """welford.cuh:73-77 : (mean, m2, n) = (0, 0, 0)."""
    return (0.0, 0.0, 0)


def welford_update(acc, x):
    """One-sample update, welford.cuh:62-70."""
    mean, m2, n = acc
    d = x - mean
    mean_new = mean + d / (n + 1)
    m2_new = m2 + d * (x - mean_new)
    return (mean_new, m2_new, n + 1)


def welford_merge(a, b):
    """Chan/Golub/LeVeque pairwise merge, welford.cuh:80-97 (n==0 operands
    are identities, :81-87)."""
    if a[2] == 0:
        return b
    if b[2] == 0:
        return a
    n = a[2] + b[2]
    d = b[0] - a[0]
    mean = a[0] + d * b[2] / n
    m2 = a[1] + b[1] + d * d * a[2] * b[2] / n
    return (mean, m2, n)


def welford_rows(x2d, chunk=None):
    """Row statistics exactly the way reduce_2d_x<WelfordOp> produces them
    (normalization.cuh:22-65): per-chunk serial updates, then merges; the
    stored variance is the biased m2 / R (welford.cuh:100-103)."""
    x2d = _f64(x2d)
    rows, R = x2d.shape
    mean = np.zeros(rows, F64)
    var = np.zeros(rows, F64)
    chunk = chunk or max(1, R // 4)
    for r in range(rows):
        total = welford_init()
        for s in range(0, R, chunk):
            acc = welford_init()
            for v in x2d[r, s:s + chunk]:
                acc = welford_update(acc, float(v))
            total = welford_merge(total, acc)
        mean[r] = total[0]
        var[r] = total[1] / R
    return mean, var


# --------------------------------------------------------------------------
# BatchNormalization
# --------------------------------------------------------------------------
def _bn_view(x, axis):
    x = _f64(x)
    shape = x.shape
    size0 = int(np.prod(shape[:axis], dtype=np.int64))
    c = shape[axis]
    size2 = int(np.prod(shape[axis + 1:], dtype=np.int64))
    return x.reshape(size0, c, size2), shape


def _bc(p, c, default):
    """gamma/beta/stat vector broadcast as [1, C, 1]; None -> default
    (no_scale / no_bias: batch_normalization.cuh:321-322,344-345)."""
    if p is None:
        return np.full((1, c, 1), default, F64)
    return _f64(p).reshape(1, c, 1)


def bn_forward_global(x, beta, gamma, rmean, rvar, axis=1, eps=1e-5):
    """Inference forward, forward_global_kernel
    (kernel/batch_normalization.cuh:332-349):
    y = (x - rm) * gamma / sqrt(rv + eps) + beta."""
    x3, shape = _bn_view(x, axis)
    c = x3.shape[1]
    y = (x3 - _bc(rmean, c, 0)) * _bc(gamma, c, 1) / np.sqrt(_bc(rvar, c, 1) + eps) \
        + _bc(beta, c, 0)
    return y.reshape(shape)


def bn_forward_batch(x, beta, gamma, rmean, rvar, axis=1, decay_rate=0.9,
                     eps=1e-5):
    """Training forward (kernel/batch_normalization.cuh:278-325):
    biased batch variance; running mean/var updated with decay_rate, the
    running variance with the unbiased factor N/(N-1) (:292-302, svar passed
    at generic/kernel/batch_normalization.cu:99).
    Returns y, mean[C], var[C], new_rmean, new_rvar (the latter two None when
    rmean/rvar is None, i.e. recompute with update_inputs=false,
    batch_normalization.cu:98-106)."""
    x3, shape = _bn_view(x, axis)
    c = x3.shape[1]
    n = x3.shape[0] * x3.shape[2]
    mean = x3.mean(axis=(0, 2))
    var = ((x3 - mean.reshape(1, c, 1)) ** 2).mean(axis=(0, 2))
    y = (x3 - mean.reshape(1, c, 1)) * _bc(gamma, c, 1) \
        / np.sqrt(var.reshape(1, c, 1) + eps) + _bc(beta, c, 0)
    new_rm = new_rv = None
    if rmean is not None:
        new_rm = decay_rate * _f64(rmean).reshape(c) + (1 - decay_rate) * mean
    if rvar is not None:
        unbiased = var * (n / (n - 1)) if n > 1 else var * np.inf
        new_rv = decay_rate * _f64(rvar).reshape(c) + (1 - decay_rate) * unbiased
    return y.reshape(shape), mean, var, new_rm, new_rv


def bn_backward_batch(x, dy, gamma, mean, var, axis=1, eps=1e-5, dmean=None,
                      dvar=None):
    """Training backward (kernel/batch_normalization.cuh:402-469,502-540):
      dvar_c  = sum(dy*g*(x-m)) * (-1/2) (v+eps)^(-3/2) + dv
      dmean_c = sum(dy*g) * (-1/sqrt(v+eps)) + dvar_c * (-2) * sum(x-m)/N + dm
      dx      = dy*g/sqrt(v+eps) + dvar_c*2(x-m)/N + dmean_c/N
      dgamma  = sum(dy*(x-m))/sqrt(v+eps),  dbeta = sum(dy)
    dm/dv are the gradients w.r.t. the mean/var outputs, present only in the
    3-output form (batch_normalization.cu:270-275).  Returns the gradient
    CONTRIBUTIONS (the reference adds them onto zeroed or accumulated
    buffers, batch_normalization.cu:263-266,293-297)."""
    x3, shape = _bn_view(x, axis)
    dy3, _ = _bn_view(dy, axis)
    c = x3.shape[1]
    n = x3.shape[0] * x3.shape[2]
    m = _f64(mean).reshape(1, c, 1)
    v = _f64(var).reshape(1, c, 1)
    g = _bc(gamma, c, 1)
    inv = 1.0 / np.sqrt(v + eps)
    xc = x3 - m
    s_dyg = (dy3 * g).sum(axis=(0, 2), keepdims=True)
    s_dygx = (dy3 * g * xc).sum(axis=(0, 2), keepdims=True)
    s_xc = xc.sum(axis=(0, 2), keepdims=True)
    dv = s_dygx * (-0.5) * (v + eps) ** (-1.5)
    if dvar is not None:
        dv = dv + _f64(dvar).reshape(1, c, 1)
    dm = s_dyg * (-inv) + dv * (-2.0) * s_xc / n
    if dmean is not None:
        dm = dm + _f64(dmean).reshape(1, c, 1)
    dx = dy3 * g * inv + dv * 2.0 * xc / n + dm / n
    dgamma = (dy3 * xc).sum(axis=(0, 2)) * inv.reshape(c)
    dbeta = dy3.sum(axis=(0, 2))
    return dx.reshape(shape), dgamma, dbeta


def bn_backward_global(x, dy, gamma, rmean, rvar, axis=1, eps=1e-5):
    """Inference-mode backward.  The reference delegates this to the absent
    NNabla core (batch_normalization.cu:209-210); this is the textbook
    gradient of bn_forward_global with the running statistics held constant
    ("convention unpinned", checked against torch eval-mode autograd)."""
    x3, shape = _bn_view(x, axis)
    dy3, _ = _bn_view(dy, axis)
    c = x3.shape[1]
    inv = 1.0 / np.sqrt(_bc(rvar, c, 1) + eps)
    dx = dy3 * _bc(gamma, c, 1) * inv
    dgamma = (dy3 * (x3 - _bc(rmean, c, 0)) * inv).sum(axis=(0, 2))
    dbeta = dy3.sum(axis=(0, 2))
    return dx.reshape(shape), dgamma, dbeta


# --------------------------------------------------------------------------
# BatchNormalization statistics of a batch split over several workers
# --------------------------------------------------------------------------
def syncbn_merge_stats(means, variances, counts, rmean=None, rvar=None,
                       decay_rate=0.9):
    """batch_norm_reduce_statistics_kernel (kernel/sync_batch_normalization.cuh:
    448-487): per channel, fold the workers' (mean, biased var, count) in
    worker order,
      var_n += v*count + (avg - m)^2 * n*count/(n+count)
      avg    = (n*avg + count*m)/(n+count);  n += count
    mean = avg, var = var_n/n; running var with var_n/(n-1).
    means, variances: [W, C]; counts: [W].  Returns mean, var, new_rmean,
    new_rvar."""
    means, variances = _f64(means), _f64(variances)
    counts = _f64(counts)
    c = means.shape[1]
    avg = np.zeros(c, F64)
    var_n = np.zeros(c, F64)
    n = 0.0
    for j in range(means.shape[0]):
        cnt = counts[j]
        factor = 1.0 / (n + cnt)
        var_n = var_n + variances[j] * cnt + (avg - means[j]) ** 2 * n * cnt * factor
        avg = n * factor * avg + cnt * factor * means[j]
        n += cnt
    new_rm = new_rv = None
    if rmean is not None:
        new_rm = decay_rate * _f64(rmean).reshape(c) + (1 - decay_rate) * avg
    if rvar is not None:
        new_rv = decay_rate * _f64(rvar).reshape(c) + (1 - decay_rate) * var_n / (n - 1)
    return avg, var_n / n, new_rm, new_rv


# --------------------------------------------------------------------------
# FusedBatchNormalization: y = relu(BatchNormalization(x) + z)
# --------------------------------------------------------------------------
def fused_bn_forward(x, z, beta, gamma, rmean, rvar, axis=1, decay_rate=0.9,
                     eps=1e-5, batch_stat=True):
    """BatchNormalization, then the residual add (add2.cuh:23-27) and
    max(0, .) (relu.cuh:48-52); what cudnnBatchNormalizationForwardTrainingEx
    computes with BN_ADD_ACTIVATION (cudnn/function/generic/
    fused_batch_normalization.cu:136-216).  z None: BN_ACTIVATION.
    Returns y, mean, var, new_rmean, new_rvar (statistics None when
    batch_stat is false)."""
    if batch_stat:
        y, mean, var, nrm, nrv = bn_forward_batch(x, beta, gamma, rmean, rvar,
                                                  axis, decay_rate, eps)
    else:
        y = bn_forward_global(x, beta, gamma, rmean, rvar, axis, eps)
        mean = var = nrm = nrv = None
    if z is not None:
        y = y + _f64(z)
    return np.maximum(y, 0.0), mean, var, nrm, nrv


def fused_bn_backward(x, y, dy, gamma, mean, var, axis=1, eps=1e-5,
                      batch_stat=True, dmean=None, dvar=None):
    """relu_add2_backward (function/generic/fused_batch_normalization.cu:
    47-75): g = dy where y > 0 else 0 (relu.cuh:56-62), dz = g (add2.cuh:
    30-35), then the BatchNormalization backward of g.  Returns dx, dz,
    dgamma, dbeta."""
    g = np.where(_f64(y) > 0, _f64(dy), 0.0)
    if batch_stat:
        dx, dgamma, dbeta = bn_backward_batch(x, g, gamma, mean, var, axis,
                                              eps, dmean, dvar)
    else:
        dx, dgamma, dbeta = bn_backward_global(x, g, gamma, mean, var, axis,
                                               eps)
    return dx, g, dgamma, dbeta


# --------------------------------------------------------------------------
# Row normalizations: shared algebra
# --------------------------------------------------------------------------
def _row_backward(x2, dy_g, mean, var, eps, dmean, dvar):
    """dx for one row-normalization, layer_normalization.cuh:50-95 (identical
    algebra in group_normalization.cuh:98-176 and
    instance_normalization.cuh:50-99):
      a  = (s1*mean - s2) * invstd^3 / R + 2*dvar/R
      b  = -a*mean - s1*invstd/R + dmean/R
      dx = dy*gamma*invstd + a*x + b
    with s1 = sum(dy*gamma), s2 = sum(dy*gamma*x) over the row
    (reduce_ops/layer_normalization.cuh:51-55).  x2, dy_g: [rows, R]."""
    R = x2.shape[1]
    m = mean.reshape(-1, 1)
    inv = 1.0 / np.sqrt(var.reshape(-1, 1) + eps)
    s1 = dy_g.sum(axis=1, keepdims=True)
    s2 = (dy_g * x2).sum(axis=1, keepdims=True)
    a = (s1 * m - s2) * inv ** 3 / R
    if dvar is not None:
        a = a + 2.0 * _f64(dvar).reshape(-1, 1) / R
    b = -a * m - s1 * inv / R
    if dmean is not None:
        b = b + _f64(dmean).reshape(-1, 1) / R
    return dy_g * inv + a * x2 + b


# --------------------------------------------------------------------------
# LayerNormalization
# --------------------------------------------------------------------------
def ln_forward(x, beta, gamma, outer, eps=1e-5):
    """x viewed [outer, R]; mean/var per row (biased, welford.cuh:100-103);
    y = gamma[i]*rsqrt(var+eps)*(x-mean) + beta[i]
    (layer_normalization.cuh:24-48)."""
    x = _f64(x)
    shape = x.shape
    x2 = x.reshape(outer, -1)
    R = x2.shape[1]
    mean = x2.mean(axis=1)
    var = ((x2 - mean[:, None]) ** 2).mean(axis=1)
    g = np.ones(R, F64) if gamma is None else _f64(gamma).reshape(R)
    b = np.zeros(R, F64) if beta is None else _f64(beta).reshape(R)
    y = g * (x2 - mean[:, None]) / np.sqrt(var[:, None] + eps) + b
    return y.reshape(shape), mean, var


def ln_backward(x, dy, gamma, mean, var, outer, eps=1e-5, dmean=None,
                dvar=None):
    """layer_normalization.cuh:50-120: dx as _row_backward;
    dbeta[i] = sum_b dy, dgamma[i] = sum_b dy*(x-mean_b)*invstd_b (:97-120)."""
    x = _f64(x)
    shape = x.shape
    x2 = x.reshape(outer, -1)
    dy2 = _f64(dy).reshape(outer, -1)
    R = x2.shape[1]
    mean = _f64(mean).reshape(outer)
    var = _f64(var).reshape(outer)
    g = np.ones(R, F64) if gamma is None else _f64(gamma).reshape(R)
    dx = _row_backward(x2, dy2 * g, mean, var, eps, dmean, dvar)
    inv = 1.0 / np.sqrt(var[:, None] + eps)
    dgamma = (dy2 * (x2 - mean[:, None]) * inv).sum(axis=0)
    dbeta = dy2.sum(axis=0)
    return dx.reshape(shape), dgamma, dbeta


# --------------------------------------------------------------------------
# GroupNormalization  (x viewed [N, C, spatial], per-channel gamma/beta)
# --------------------------------------------------------------------------
def gn_forward(x, beta, gamma, n, c, num_groups, eps=1e-5):
    """Welford per (n, g) over (C/G)*spatial elements, then
    a = gamma_c * rsqrt(var+eps), b = beta_c - mean*a, y = a*x + b
    (group_normalization.cuh:32-73; sizes group_normalization.cu:57-62).
    Returns y, mean[N*G], var[N*G]."""
    x = _f64(x)
    shape = x.shape
    xg = x.reshape(n * num_groups, -1)
    mean = xg.mean(axis=1)
    var = ((xg - mean[:, None]) ** 2).mean(axis=1)
    cpg = c // num_groups
    x3 = x.reshape(n, c, -1)
    g = np.ones(c, F64) if gamma is None else _f64(gamma).reshape(c)
    b = np.zeros(c, F64) if beta is None else _f64(beta).reshape(c)
    inv = np.repeat((1.0 / np.sqrt(var + eps)).reshape(n, num_groups), cpg, axis=1)
    mu = np.repeat(mean.reshape(n, num_groups), cpg, axis=1)
    a = g[None, :] * inv
    bb = b[None, :] - mu * a
    y = a[:, :, None] * x3 + bb[:, :, None]
    return y.reshape(shape), mean, var


def gn_backward(x, dy, gamma, mean, var, n, c, num_groups, eps=1e-5,
                dmean=None, dvar=None):
    """group_normalization.cuh:75-206: per-(n,c) sum_dy, sum_dyx
    (reduce_ops/group_normalization.cuh:40-68); per-(n,g) factors with
    S1 = sum_c sum_dy*gamma_c, S2 = sum_c sum_dyx*gamma_c (:98-149);
    dx = gamma_c*invstd*dy + f1*x + f2 (:151-176);
    dbeta_c = sum_n sum_dy, dgamma_c = sum_n (sum_dyx - sum_dy*mean)*invstd
    (:178-206)."""
    x = _f64(x)
    shape = x.shape
    cpg = c // num_groups
    x3 = x.reshape(n, c, -1)
    dy3 = _f64(dy).reshape(n, c, -1)
    g = np.ones(c, F64) if gamma is None else _f64(gamma).reshape(c)
    mean = _f64(mean).reshape(n * num_groups)
    var = _f64(var).reshape(n * num_groups)
    dyg = (dy3 * g[None, :, None]).reshape(n * num_groups, -1)
    dx = _row_backward(x.reshape(n * num_groups, -1), dyg, mean, var, eps,
                       dmean, dvar)
    sum_dy = dy3.sum(axis=2)
    sum_dyx = (dy3 * x3).sum(axis=2)
    mu = np.repeat(mean.reshape(n, num_groups), cpg, axis=1)
    inv = np.repeat((1.0 / np.sqrt(var + eps)).reshape(n, num_groups), cpg, axis=1)
    dbeta = sum_dy.sum(axis=0)
    dgamma = ((sum_dyx - sum_dy * mu) * inv).sum(axis=0)
    return dx.reshape(shape), dgamma, dbeta


# --------------------------------------------------------------------------
# InstanceNormalization  (x viewed [N, C, spatial])
# --------------------------------------------------------------------------
def in_forward(x, beta, gamma, n, c, eps=1e-5):
    """Per-(n,c) row statistics; gamma/beta either per channel (broadcast
    over the batch, index outer_idx % C) or per (n,c) (index outer_idx)
    (instance_normalization.cuh:24-48).  A gamma/beta of size C is the
    broadcast form, of size N*C the per-sample form.
    Returns y, mean[N*C], var[N*C]."""
    x = _f64(x)
    shape = x.shape
    x2 = x.reshape(n * c, -1)
    mean = x2.mean(axis=1)
    var = ((x2 - mean[:, None]) ** 2).mean(axis=1)

    def expand(p, default):
        if p is None:
            return np.full(n * c, default, F64)
        p = _f64(p).reshape(-1)
        return np.tile(p, n) if p.size == c and n * c != c else p.reshape(n * c)

    g = expand(gamma, 1.0)
    b = expand(beta, 0.0)
    y = g[:, None] * (x2 - mean[:, None]) / np.sqrt(var[:, None] + eps) + b[:, None]
    return y.reshape(shape), mean, var


def in_backward(x, dy, gamma, mean, var, n, c, eps=1e-5, dmean=None,
                dvar=None, bc_gamma=True, bc_beta=True):
    """instance_normalization.cuh:50-121: factors with scalar per-row gamma;
    per-(n,c) dbeta = sum_dy, dgamma = (sum_dyx - sum_dy*mean)*invstd; summed
    over the batch when the parameter is broadcast
    (instance_normalization.cu:427-464)."""
    x = _f64(x)
    shape = x.shape
    x2 = x.reshape(n * c, -1)
    dy2 = _f64(dy).reshape(n * c, -1)
    mean = _f64(mean).reshape(n * c)
    var = _f64(var).reshape(n * c)
    if gamma is None:
        g = np.ones(n * c, F64)
    else:
        g = _f64(gamma).reshape(-1)
        g = np.tile(g, n) if bc_gamma else g.reshape(n * c)
    dx = _row_backward(x2, dy2 * g[:, None], mean, var, eps, dmean, dvar)
    inv = 1.0 / np.sqrt(var + eps)
    sum_dy = dy2.sum(axis=1)
    sum_dyx = (dy2 * x2).sum(axis=1)
    dbeta = sum_dy
    dgamma = sum_dyx * inv - sum_dy * mean * inv
    if bc_beta:
        dbeta = dbeta.reshape(n, c).sum(axis=0)
    if bc_gamma:
        dgamma = dgamma.reshape(n, c).sum(axis=0)
    return dx.reshape(shape), dgamma, dbeta
