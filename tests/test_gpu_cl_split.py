"""Channel-last Group/InstanceNormalization through the split kernels: a block owns
whole 128-byte lines of a range of positions and the blocks of a sample
exchange partial sums (each partial one {value, epoch} word).  Parity against
the oracle on the transposed tensor; the path a block takes when a partner's
word does not arrive (it computes that partner's part itself) is forced by
allowing no polls and must give bit-identical results; host threads on their
own streams share the exchange array; a captured graph must not take these
kernels (an epoch would be replayed) and still be right."""
import threading

import numpy as np
import pytest
import torch

from _util import assert_close, dtype_name, load_package, rounded, to_dev, to_np
from oracle import norm_ref as R

pytestmark = pytest.mark.gpu
K = load_package()
F32, F16 = torch.float32, torch.float16


def f32(a):
    return np.asarray(a, np.float32).astype(np.float64)


@pytest.fixture(autouse=True)
def _default_knobs():
    K.tune_reset()
    yield
    K.tune_reset()
    K.check(K.lib().nblahip_profile_enable(0))


def to_cf(a):
    return np.ascontiguousarray(np.moveaxis(a, -1, 1))


def to_cl(a):
    return np.ascontiguousarray(np.moveaxis(a, 1, -1))


def make(n, sp, c, dtype, seed):
    rng = np.random.default_rng(seed)
    shape = (n,) + sp + (c,)
    x = rounded(rng.standard_normal(shape) * 1.5 + rng.uniform(-2, 2, (n,) + (1,) * len(sp) + (c,)), dtype)
    dy = rounded(rng.standard_normal(shape), dtype)
    return x, dy, f32(rng.uniform(0.5, 1.5, c)), f32(rng.standard_normal(c) * 0.1)


def ran(names):
    return "cl_split_fwd_kernel" in names and "cl_split_bwd_kernel" in names


# (n, spatial, c, groups): ragged last block, 1 / 2 / 4 / 8 vectors per group,
# one block per (sample, tile), planes up to the 16 x 1024 positions the largest
# block shape covers, several column tiles
SHAPES = [(3, (33, 33), 64, 8), (2, (20, 20), 128, 4), (5, (9, 9), 64, 1), (2, (70, 70), 64, 8),
          (1, (127, 129), 64, 2), (2, (100, 100), 32, 4), (4, (16, 16), 512, 16), (2, (7,), 64, 8),
          (1, (300,), 192, 12),
          # many (sample, block) rows of pairs behind dgamma / dbeta
          (40, (20, 20), 64, 8), (70, (6, 6), 128, 16)]


@pytest.mark.parametrize("n,sp,c,groups", SHAPES)
@pytest.mark.parametrize("dtype", [F32, F16])
def test_split_kernels_match_the_oracle_with_and_without_the_exchange(n, sp, c, groups, dtype):
    dn = dtype_name(dtype)
    vec = 8 if dtype == F16 else 4
    cpg = c // groups
    eligible = c % (8 * vec) == 0 and cpg % vec == 0 and cpg // vec in (1, 2, 4, 8)
    x, dy, g, b = make(n, sp, c, dtype, 21)
    xt, dyt = to_cf(x), to_cf(dy)
    y_r, m_r, v_r = R.gn_forward(xt, b, g, n, c, groups, 1e-5)
    dx_r, dg_r, db_r = R.gn_backward(xt, dyt, g, m_r, v_r, n, c, groups, 1e-5)
    xd, dyd, gd, bd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(b)

    def run():
        K.check(K.lib().nblahip_profile_enable(64))
        y, m, v = K.gn_forward(xd, bd, gd, groups, 1e-5, channel_last=True)
        dx, dgam, dbet = K.gn_backward(xd, dyd, gd, m, v, groups, 1e-5, channel_last=True)
        torch.cuda.synchronize()
        names = K.profile_kernels()
        K.check(K.lib().nblahip_profile_enable(0))
        return [y, m, v, dx, dgam, dbet], names

    out, names = run()
    assert ran(names) == eligible, names
    y, m, v, dx, dgam, dbet = out
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(y), to_cl(y_r.reshape(xt.shape)), dn, "y", "y")
    assert_close(to_np(dx), to_cl(dx_r.reshape(xt.shape)), dn, "grad", "dx")
    assert_close(to_np(dgam), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(dbet), db_r, dn, "pgrad", "dbeta")
    if not eligible:
        return
    # no poll allowed: every block recomputes all its partners' parts, in the
    # arithmetic the partners use, so not a bit may change
    K.tune_set("XCHG_SPIN", 0)
    out2, names2 = run()
    assert ran(names2)
    for a_, b_ in zip(out, out2):
        assert torch.equal(a_, b_)
    # and twice the same
    K.tune_reset()
    out3, _ = run()
    for a_, b_ in zip(out, out3):
        assert torch.equal(a_, b_)


@pytest.mark.parametrize("kind", ["offset", "outlier_first", "constant"])
@pytest.mark.parametrize("groups", [8, 64])
@pytest.mark.parametrize("dtype", [F32, F16])
def test_one_pass_statistics_on_hard_data(kind, groups, dtype):
    """The statistics shift by each thread's own mean: a mean far
    from zero, one huge value at the first position of every channel (1000
    deviations off everything else its thread holds) and constant data
    (variance 0 to rounding) must come out within the statistics' tolerance; groups of 8 channels and
    instances."""
    dn = dtype_name(dtype)
    n, sp, c = 3, (40, 40), 64
    rng = np.random.default_rng(78)
    shape = (n,) + sp + (c,)
    if kind == "offset":
        x = rng.standard_normal(shape) + (300.0 if dtype == F32 else 40.0)
    elif kind == "outlier_first":
        x = rng.standard_normal(shape)
        x[:, 0, 0, :] = 1000.0
    else:
        x = np.full(shape, 3.25)
    x = rounded(x, dtype)
    xt = to_cf(x)
    K.check(K.lib().nblahip_profile_enable(8))
    if groups == c:
        y_r, m_r, v_r = R.in_forward(xt, None, None, n, c, 1e-5)
        y, m, v = K.in_forward(to_dev(x, dtype), None, None, 1e-5, channel_last=True)
    else:
        y_r, m_r, v_r = R.gn_forward(xt, None, None, n, c, groups, 1e-5)
        y, m, v = K.gn_forward(to_dev(x, dtype), None, None, groups, 1e-5, channel_last=True)
    torch.cuda.synchronize()
    names = K.profile_kernels()
    K.check(K.lib().nblahip_profile_enable(0))
    assert names == ["cl_split_fwd_kernel"], names
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    if kind == "constant":
        assert float(v.abs().max()) < 1e-10
    # (at an offset of 300 a float x is itself only known to 3e-5, and so is x - mean)
    assert_close(to_np(y), to_cl(y_r.reshape(xt.shape)), dn, "y", "y",
                 scale=10.0 if kind == "offset" and dtype == F32 else 1.0 if kind == "constant" else None)


@pytest.mark.parametrize("spin", [64, 0])
def test_split_flags(spin):
    """no_scale/no_bias, dmean/dvar, accumulation onto dx/dgamma/dbeta, parameter
    gradients only, dx only."""
    K.tune_set("XCHG_SPIN", spin)
    n, sp, c, groups = 3, (24, 24), 64, 4
    rng = np.random.default_rng(9)
    x, dy, g, b = make(n, sp, c, F32, 31)
    xt, dyt = to_cf(x), to_cf(dy)
    xd, dyd = to_dev(x), to_dev(dy)
    y_r, m_r, v_r = R.gn_forward(xt, None, None, n, c, groups, 1e-5)
    K.check(K.lib().nblahip_profile_enable(64))
    y, m, v = K.gn_forward(xd, None, None, groups, 1e-5, channel_last=True)
    assert_close(to_np(y), to_cl(y_r.reshape(xt.shape)), "f32", "y", "y no params")
    dx_r, _, _ = R.gn_backward(xt, dyt, None, m_r, v_r, n, c, groups, 1e-5)
    dx, _, _ = K.gn_backward(xd, dyd, None, m, v, groups, 1e-5, need=(True, False, False),
                             channel_last=True)
    assert_close(to_np(dx), to_cl(dx_r.reshape(xt.shape)), "f32", "grad", "dx no params")
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
    _, dgam, dbet = K.gn_backward(xd, dyd, to_dev(g), m, v, groups, 1e-5, dmean=to_dev(dm),
                                  dvar=to_dev(dv), need=(False, True, True), channel_last=True)
    assert_close(to_np(dgam), dg_r, "f32", "pgrad", "dgamma only")
    assert_close(to_np(dbet), db_r, "f32", "pgrad", "dbeta only")
    _, dgam, none = K.gn_backward(xd, dyd, to_dev(g), m, v, groups, 1e-5, dmean=to_dev(dm),
                                  dvar=to_dev(dv), need=(True, True, False), channel_last=True)
    assert none is None
    assert_close(to_np(dgam), dg_r, "f32", "pgrad", "dgamma without dbeta")
    torch.cuda.synchronize()
    assert ran(K.profile_kernels())


def test_threads_on_their_own_streams_share_the_exchange_array():
    """Eight threads, each repeating its own forward+backward on its own
    stream: every call has its own epoch and region, overlapping calls never
    read each other's words, and each result equals the single-threaded one
    bit for bit."""
    def work(seed):
        gen = torch.Generator(device="cuda").manual_seed(seed)
        x = torch.randn(4, 40, 40, 128, device="cuda", generator=gen).half()
        dy = torch.randn(4, 40, 40, 128, device="cuda", generator=gen).half()
        gamma = torch.rand(128, device="cuda", generator=gen) + 0.5
        beta = torch.randn(128, device="cuda", generator=gen)
        y, m, v = K.gn_forward(x, beta, gamma, 16, 1e-5, channel_last=True)
        return [y, m, v, *K.gn_backward(x, dy, gamma, m, v, 16, 1e-5, channel_last=True)]

    want = [[t.clone() for t in work(200 + i)] for i in range(8)]
    torch.cuda.synchronize()
    got, errors = [None] * 8, []

    def run(i):
        try:
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                for _ in range(10):
                    out = work(200 + i)
                s.synchronize()
            got[i] = out
        except Exception as e:  # noqa: BLE001 - reported below
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=run, args=(i,)) for i in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for w, g_ in zip(want, got):
        for a_, b_ in zip(w, g_):
            assert torch.equal(a_, b_)


def test_a_captured_graph_takes_the_other_kernels_and_replays_correctly():
    shape, c, groups = (4, 24, 24, 64), 64, 8
    x = torch.empty(shape, device="cuda", dtype=F16)
    dy = torch.empty_like(x)
    gamma = torch.rand(c, device="cuda") + 0.5
    beta = torch.randn(c, device="cuda")

    def eager(xi, dyi):
        y, m, v = K.gn_forward(xi, beta, gamma, groups, 1e-5, channel_last=True)
        return [y, m, v, *K.gn_backward(xi, dyi, gamma, m, v, groups, 1e-5, channel_last=True)]

    x.normal_()
    dy.normal_()
    eager(x, dy)
    torch.cuda.synchronize()
    st = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(st):
        with torch.cuda.graph(graph, stream=st):
            outs = eager(x, dy)
    torch.cuda.synchronize()
    for rep in range(3):
        xi = (torch.randn(shape, device="cuda") * (rep + 1)).half()
        dyi = torch.randn(shape, device="cuda").half()
        split = [t.clone() for t in eager(xi, dyi)]          # the split kernels, eagerly
        K.tune_set("GN_CL_SPLIT", 0)
        want = [t.clone() for t in eager(xi, dyi)]           # the kernels a capture takes
        K.tune_reset()
        x.copy_(xi)
        dy.copy_(dyi)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for a_, b_ in zip(want, outs):
            assert torch.equal(a_, b_), rep
        for a_, b_ in zip(split, outs):                      # same function, other summation order
            torch.testing.assert_close(a_.float(), b_.float(), rtol=2e-2, atol=2e-2)


IN_SHAPES = [(3, (33, 33), 64), (2, (70, 70), 64), (5, (9, 9), 128), (2, (100, 100), 32), (2, (7,), 64),
             (1, (127, 129), 64), (4, (16, 16), 256)]


@pytest.mark.parametrize("n,sp,c", IN_SHAPES)
@pytest.mark.parametrize("dtype", [F32, F16])
def test_instances_through_the_split_kernels(n, sp, c, dtype):
    dn = dtype_name(dtype)
    eligible = c % (64 if dtype == F16 else 32) == 0
    x, dy, g, b = make(n, sp, c, dtype, 23)
    xt, dyt = to_cf(x), to_cf(dy)
    y_r, m_r, v_r = R.in_forward(xt, b, g, n, c, 1e-5)
    dx_r, dg_r, db_r = R.in_backward(xt, dyt, g, m_r, v_r, n, c, 1e-5)
    xd, dyd, gd, bd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(b)

    def run():
        K.check(K.lib().nblahip_profile_enable(64))
        y, m, v = K.in_forward(xd, bd, gd, 1e-5, channel_last=True)
        dx, dgam, dbet = K.in_backward(xd, dyd, gd, m, v, 1e-5, channel_last=True)
        torch.cuda.synchronize()
        names = K.profile_kernels()
        K.check(K.lib().nblahip_profile_enable(0))
        return [y, m, v, dx, dgam, dbet], names

    out, names = run()
    assert ran(names) == eligible, names
    y, m, v, dx, dgam, dbet = out
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(y), to_cl(y_r.reshape(xt.shape)), dn, "y", "y")
    assert_close(to_np(dx), to_cl(dx_r.reshape(xt.shape)), dn, "grad", "dx")
    assert_close(to_np(dgam), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(dbet), db_r, dn, "pgrad", "dbeta")
    if not eligible:
        return
    K.tune_set("XCHG_SPIN", 0)     # every partner's part recomputed: not a bit may change
    out2, names2 = run()
    assert ran(names2)
    for a_, b_ in zip(out, out2):
        assert torch.equal(a_, b_)


def test_instance_flags_through_the_split_kernels():
    """dmean/dvar, accumulation, parameter gradients only, no parameters."""
    n, sp, c = 3, (24, 24), 64
    rng = np.random.default_rng(10)
    x, dy, g, b = make(n, sp, c, F32, 33)
    xt, dyt = to_cf(x), to_cf(dy)
    xd, dyd = to_dev(x), to_dev(dy)
    K.check(K.lib().nblahip_profile_enable(64))
    y_r, m_r, v_r = R.in_forward(xt, None, None, n, c, 1e-5)
    y, m, v = K.in_forward(xd, None, None, 1e-5, channel_last=True)
    assert_close(to_np(y), to_cl(y_r.reshape(xt.shape)), "f32", "y", "y no params")
    dm, dv = f32(rng.standard_normal(n * c)), f32(rng.standard_normal(n * c))
    y_r, m_r, v_r = R.in_forward(xt, b, g, n, c, 1e-5)
    dx_r, dg_r, db_r = R.in_backward(xt, dyt, g, m_r, v_r, n, c, 1e-5, dmean=dm, dvar=dv)
    y, m, v = K.in_forward(xd, to_dev(b), to_dev(g), 1e-5, channel_last=True)
    pre_dx = rng.standard_normal(x.shape).astype(np.float32)
    pre_g = rng.standard_normal(c).astype(np.float32)
    dxd, dgd = to_dev(pre_dx), to_dev(pre_g)
    K.in_backward(xd, dyd, to_dev(g), m, v, 1e-5, dmean=to_dev(dm), dvar=to_dev(dv), dx=dxd,
                  dgamma=dgd, accum=(True, True, False), channel_last=True)
    assert_close(to_np(dxd), to_cl(dx_r.reshape(xt.shape)) + pre_dx, "f32", "grad", "dx accum")
    assert_close(to_np(dgd), dg_r + pre_g, "f32", "pgrad", "dgamma accum")
    _, dgam, dbet = K.in_backward(xd, dyd, to_dev(g), m, v, 1e-5, dmean=to_dev(dm), dvar=to_dev(dv),
                                  need=(False, True, True), channel_last=True)
    assert_close(to_np(dgam), dg_r, "f32", "pgrad", "dgamma only")
    assert_close(to_np(dbet), db_r, "f32", "pgrad", "dbeta only")
    torch.cuda.synchronize()
    assert ran(K.profile_kernels())


def test_epoch_wrap_and_ring_end():
    """The per-launch epoch is a 32-bit counter: walked across its wrap (the
    library then clears the exchange array and starts over) and, with launches
    of many exchange words, several times round the ring, results stay
    bit-identical to the first call and the exchanging kernels keep running."""
    n, sp, c, groups = 16, (64, 64), 256, 32       # 16 x 4 x 16 blocks' words per launch
    x, dy, g, b = make(n, sp, c, F16, 77)
    xd, dyd, gd, bd = to_dev(x, F16), to_dev(dy, F16), to_dev(g), to_dev(b)

    def run():
        y, m, v = K.gn_forward(xd, bd, gd, groups, 1e-5, channel_last=True)
        dx, dgam, dbet = K.gn_backward(xd, dyd, gd, m, v, groups, 1e-5, channel_last=True)
        return [y, m, v, dx, dgam, dbet]

    first = run()
    K.check(K.lib().nblahip_xchg_set_epoch(0xFFFFFFFF - 5))
    K.check(K.lib().nblahip_profile_enable(256))
    for _ in range(12):                              # 24 launches: across the wrap
        out = run()
        for a_, b_ in zip(first, out):
            assert torch.equal(a_, b_)
    torch.cuda.synchronize()
    names = K.profile_kernels()
    K.check(K.lib().nblahip_profile_enable(0))
    assert ran(names), names
    # many launches with large regions: round the ring more than once
    big = make(64, (32, 32), 512, F16, 78)
    bx, bdy, bg, bb = to_dev(big[0], F16), to_dev(big[1], F16), to_dev(big[2]), to_dev(big[3])
    ref = None
    for _ in range(40):
        y, m, v = K.in_forward(bx, bb, bg, 1e-5, channel_last=True)
        if ref is None:
            ref = (y.clone(), m.clone(), v.clone())
        else:
            assert torch.equal(y, ref[0]) and torch.equal(m, ref[1]) and torch.equal(v, ref[2])
    out = run()
    for a_, b_ in zip(first, out):
        assert torch.equal(a_, b_)
