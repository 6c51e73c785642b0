"""Golden vectors of tests/golden/*.npz (PyTorch CPU float64 operators and
autograd, written by tests/golden/make_fixtures.py; the reference tree holds no
stored vectors for these functions): the oracle must reproduce them to float64
rounding, the HIP path to the stated tolerances."""
import glob
import os

import numpy as np
import pytest

from _util import assert_close, load_package
from oracle import norm_ref as R

HERE = os.path.dirname(os.path.abspath(__file__))
FILES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))
NAMES = [os.path.splitext(os.path.basename(f))[0] for f in FILES]


def load(name):
    with np.load(os.path.join(HERE, "golden", name + ".npz"), allow_pickle=False) as z:
        d = {k: z[k] for k in z.files}
    for k in ("kind", "dtype"):
        d[k] = str(d[k])
    for k in ("x", "dy", "gamma", "beta", "rmean", "rvar", "dmean", "dvar"):
        if k in d:
            d[k] = d[k].astype(np.float64)
    d["eps"] = float(d["eps"])
    d["stat_grads"] = bool(int(d["stat_grads"]))
    return d


def test_fixture_inventory():
    kinds = {load(n)["kind"] for n in NAMES}
    assert kinds == {"bn", "ln", "gn"} and len(NAMES) >= 22


def close64(got, ref, name):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    assert got.reshape(-1).shape == ref.reshape(-1).shape, name
    scale = max(1.0, float(np.abs(ref).max()))
    err = float(np.abs(got.reshape(-1) - ref.reshape(-1)).max())
    assert err <= 1e-9 * scale, f"{name}: max error {err:.3e} (scale {scale:.3g})"


def run(d, ops, check):
    """Forward, backward (and BN inference) of one fixture through `ops` (the
    oracle's functions on numpy arrays or the C-ABI binding on device tensors);
    check(name, got, expected, kind) compares."""
    dm = d["dmean"] if d["stat_grads"] else None
    dv = d["dvar"] if d["stat_grads"] else None
    eps = d["eps"]
    if d["kind"] == "bn":
        axis = int(d["axis"])
        y, m, v, rm, rv = ops.bn_forward(d["x"], d["beta"], d["gamma"], d["rmean"], d["rvar"], axis,
                                         float(d["decay_rate"]), eps)
        check("y", y, d["y"], "y")
        check("mean", m, d["mean"], "stat")
        check("var", v, d["var"], "stat")
        check("running mean", rm, d["rmean_out"], "stat")
        check("running var", rv, d["rvar_out"], "stat")
        dx, dg, db = ops.bn_backward(d["x"], d["dy"], d["gamma"], m, v, axis, eps, dm, dv)
        check("inference y", ops.bn_inference(d["x"], d["beta"], d["gamma"], d["rmean"], d["rvar"],
                                              axis, eps), d["y_inference"], "y")
    elif d["kind"] == "ln":
        outer = d["x"].shape[0]
        y, m, v = ops.ln_forward(d["x"], d["beta"], d["gamma"], outer, eps)
        check("y", y, d["y"], "y")
        check("mean", m, d["mean"], "stat")
        check("var", v, d["var"], "stat")
        dx, dg, db = ops.ln_backward(d["x"], d["dy"], d["gamma"], m, v, outer, eps, dm, dv)
    else:
        groups = int(d["groups"])
        y, m, v = ops.gn_forward(d["x"], d["beta"], d["gamma"], groups, eps)
        check("y", y, d["y"], "y")
        check("mean", m, d["mean"], "stat")
        check("var", v, d["var"], "stat")
        dx, dg, db = ops.gn_backward(d["x"], d["dy"], d["gamma"], m, v, groups, eps, dm, dv)
    check("dx", dx, d["dx"], "grad")
    check("dgamma", dg, d["dgamma"], "pgrad")
    check("dbeta", db, d["dbeta"], "pgrad")


class OracleOps:
    """The float64 oracle on numpy arrays."""

    @staticmethod
    def bn_forward(x, b, g, rm, rv, axis, decay, eps):
        return R.bn_forward_batch(x, b, g, rm, rv, axis, decay, eps)

    @staticmethod
    def bn_backward(x, dy, g, m, v, axis, eps, dm, dv):
        return R.bn_backward_batch(x, dy, g, m, v, axis, eps, dm, dv)

    @staticmethod
    def bn_inference(x, b, g, rm, rv, axis, eps):
        return R.bn_forward_global(x, b, g, rm, rv, axis, eps)

    @staticmethod
    def ln_forward(x, b, g, outer, eps):
        return R.ln_forward(x, b, g, outer, eps)

    @staticmethod
    def ln_backward(x, dy, g, m, v, outer, eps, dm, dv):
        return R.ln_backward(x, dy, g, m, v, outer, eps, dm, dv)

    @staticmethod
    def gn_forward(x, b, g, groups, eps):
        n, c = x.shape[0], x.shape[1]
        if groups == c:
            return R.in_forward(x, b, g, n, c, eps)
        return R.gn_forward(x, b, g, n, c, groups, eps)

    @staticmethod
    def gn_backward(x, dy, g, m, v, groups, eps, dm, dv):
        n, c = x.shape[0], x.shape[1]
        if groups == c:
            return R.in_backward(x, dy, g, m, v, n, c, eps, dm, dv)
        return R.gn_backward(x, dy, g, m, v, n, c, groups, eps, dm, dv)


@pytest.mark.parametrize("name", NAMES)
def test_oracle_reproduces_golden(name):
    d = load(name)
    run(d, OracleOps, lambda what, got, ref, kind: close64(got, ref, f"{name} {what}"))


class HipOps:
    """The HIP path through the C-ABI binding; inputs go to the device in the
    fixture's storage dtype, parameters and statistics in float32."""

    def __init__(self, dtype):
        import torch
        self.K = load_package()
        self.torch = torch
        self.dt = torch.float16 if dtype == "f16" else torch.float32

    def dev(self, a, data=False):
        t = self.torch.from_numpy(np.ascontiguousarray(a))
        return t.to(self.dt if data else self.torch.float32).cuda()

    def bn_forward(self, x, b, g, rm, rv, axis, decay, eps):
        rmd, rvd = self.dev(rm), self.dev(rv)
        y, m, v = self.K.bn_forward_batch(self.dev(x, True), self.dev(b), self.dev(g), rmd, rvd, axis,
                                          decay, eps)
        return y, m, v, rmd, rvd

    def bn_backward(self, x, dy, g, m, v, axis, eps, dm, dv):
        return self.K.bn_backward(self.dev(x, True), self.dev(dy, True), self.dev(g), m, v, axis, eps,
                                  dmean=None if dm is None else self.dev(dm),
                                  dvar=None if dv is None else self.dev(dv))

    def bn_inference(self, x, b, g, rm, rv, axis, eps):
        return self.K.bn_forward_global(self.dev(x, True), self.dev(b), self.dev(g), self.dev(rm),
                                        self.dev(rv), axis, eps)

    def ln_forward(self, x, b, g, outer, eps):
        return self.K.ln_forward(self.dev(x, True), self.dev(b), self.dev(g), outer, eps)

    def ln_backward(self, x, dy, g, m, v, outer, eps, dm, dv):
        return self.K.ln_backward(self.dev(x, True), self.dev(dy, True), self.dev(g), m, v, outer, eps,
                                  dmean=None if dm is None else self.dev(dm),
                                  dvar=None if dv is None else self.dev(dv))

    def gn_forward(self, x, b, g, groups, eps):
        if groups == x.shape[1]:
            return self.K.in_forward(self.dev(x, True), self.dev(b), self.dev(g), eps)
        return self.K.gn_forward(self.dev(x, True), self.dev(b), self.dev(g), groups, eps)

    def gn_backward(self, x, dy, g, m, v, groups, eps, dm, dv):
        kw = dict(dmean=None if dm is None else self.dev(dm), dvar=None if dv is None else self.dev(dv))
        if groups == x.shape[1]:
            return self.K.in_backward(self.dev(x, True), self.dev(dy, True), self.dev(g), m, v, eps, **kw)
        return self.K.gn_backward(self.dev(x, True), self.dev(dy, True), self.dev(g), m, v, groups, eps,
                                  **kw)


@pytest.mark.gpu
@pytest.mark.parametrize("name", NAMES)
def test_hip_path_reproduces_golden(name):
    d = load(name)
    dn = d["dtype"]

    def check(what, got, ref, kind):
        assert_close(got.detach().float().cpu().numpy(), ref, dn, kind, f"{name} {what}")

    run(d, HipOps(dn), check)


class HipChannelLastOps(HipOps):
    """Group / InstanceNormalization fixtures (stored channel-first) run through
    the channel-last entry points on the transposed tensors; outputs come back
    transposed."""

    @staticmethod
    def cl(a):
        return np.ascontiguousarray(np.moveaxis(np.asarray(a), 1, -1))

    def back(self, t):
        return self.torch.movedim(t, -1, 1).contiguous()

    def gn_forward(self, x, b, g, groups, eps):
        xd = self.dev(self.cl(x), True)
        if groups == x.shape[1]:
            y, m, v = self.K.in_forward(xd, self.dev(b), self.dev(g), eps, channel_last=True)
        else:
            y, m, v = self.K.gn_forward(xd, self.dev(b), self.dev(g), groups, eps, channel_last=True)
        return self.back(y), m, v

    def gn_backward(self, x, dy, g, m, v, groups, eps, dm, dv):
        kw = dict(dmean=None if dm is None else self.dev(dm), dvar=None if dv is None else self.dev(dv),
                  channel_last=True)
        xd, dyd = self.dev(self.cl(x), True), self.dev(self.cl(dy), True)
        if groups == x.shape[1]:
            dx, dg, db = self.K.in_backward(xd, dyd, self.dev(g), m, v, eps, **kw)
        else:
            dx, dg, db = self.K.gn_backward(xd, dyd, self.dev(g), m, v, groups, eps, **kw)
        return self.back(dx), dg, db


@pytest.mark.gpu
@pytest.mark.parametrize("name", [n for n in NAMES if n.startswith(("gn_", "in_"))])
def test_hip_channel_last_reproduces_golden(name):
    d = load(name)
    dn = d["dtype"]

    def check(what, got, ref, kind):
        assert_close(got.detach().float().cpu().numpy(), ref, dn, kind, f"{name} channel-last {what}")

    run(d, HipChannelLastOps(dn), check)


# Fixtures again with the default plan of their shape switched off, so that the
# plans behind it are held to the same vectors: (fixture, knobs).
PLAN_VARIANTS = [
    ("bn_nchw_f16_7x7_planes", {"BN_ROWS": 0}),                       # channel packs / masked split reduction
    ("bn_nchw_f16_7x7_planes", {"BN_ROWS": 0, "BN_PACK": 0}),
    ("bn_nchw_f32_17x17_planes", {"BN_ROWS": 0}),                     # a channel per block, masked vectors
    ("bn_nchw_f32_17x17_planes", {"BN_ROWS": 0, "BN_MASKED_ONCHIP": 0}),
    ("bn_nchw_f32_17x17_planes", {"BN_ROWS": 0, "BN_MASKED_ONCHIP": 0, "BN_MASKED_PLANES": 0}),
    ("bn_nhwc_f16_outliers", {"BN_CL_CACHED": 0}),
    ("bn_nhwc_f16_outliers", {"BN_CL_CACHED": 0, "BN_CL_SPLIT": 0}),
    ("ln_f16_odd_hidden", {"LN_LOOSE": 0}),
    ("ln_f16_odd_hidden", {"FORCE_STREAM": 1}),
    ("in_f16_odd_planes", {"ROW_MASKED": 0}),
    ("gn_f16_odd_planes", {"ROW_MASKED": 0}),
    ("gn_f16_wide", {"FORCE_STREAM": 1}),
]


@pytest.mark.gpu
@pytest.mark.parametrize("name,knobs", PLAN_VARIANTS)
def test_hip_plan_variants_reproduce_golden(name, knobs):
    d = load(name)
    dn = d["dtype"]
    K = load_package()

    def check(what, got, ref, kind):
        assert_close(got.detach().float().cpu().numpy(), ref, dn, kind, f"{name} {knobs} {what}")

    K.tune_reset()
    for k, v in knobs.items():
        K.tune_set(k, v)
    try:
        run(d, HipOps(dn), check)
    finally:
        K.tune_reset()
