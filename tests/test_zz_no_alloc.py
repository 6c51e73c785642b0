"""nblahip_bn_fwd_train_static, the BatchNormalization training forward for
callers that cannot allocate: its split-reduction partials live in an array
inside the library instead of a caller's workspace.  Checked against
nblahip_bn_fwd_train (same kernels, same plan: the results must be equal bit
for bit) and against the float64 oracle, on two calls in a row, the second
with a smaller input, so that what the first call left in the shared array
is there when the second one runs."""
import numpy as np
import pytest

from _util import assert_close, load_package, to_np

K = load_package()

# (shape, axis, dtype name): tensors that take the split reduction, i.e. use
# the scratch array (channel-last with many rows - 96 channels, which the
# kernel that holds the tensor on the chip takes only in 64-byte column
# strips, switched off here, and 32 channels in fewer rows than it is given;
# planes with few
# channels, with the plans that hold a channel on one CU or split it over
# several blocks switched off), and a pair that does not need it (held on the
# chip, the partials travel through the exchange array): the entry point must
# agree there too.
CASES = [
    ([((64, 56, 56, 96), 3, "f16"), ((8, 28, 28, 32), 3, "f16")], True,
     {"BN_CL_GRID_STRIP_MIN_VECS": 8, "BN_CL_GRID_NARROW_MIN_ROWS": 10240}),
    ([((32, 8, 56, 56), 1, "f32"), ((32, 8, 40, 40), 1, "f32")], True,
     {"BN_CHAN_SPLIT": 0, "BN_ONCHIP": 0}),
    ([((64, 56, 56, 64), 3, "f16"), ((56, 56, 56, 64), 3, "f16")], False, {}),
]


def _inputs(shape, axis, dt, seed):
    import torch
    rng = np.random.default_rng(seed)
    c = shape[axis]
    tdt = torch.float16 if dt == "f16" else torch.float32
    x = torch.from_numpy((rng.standard_normal(shape) * 2 + 1).astype(np.float32)).to(tdt).cuda()
    g = torch.from_numpy(rng.uniform(0.5, 1.5, c).astype(np.float32)).cuda()
    b = torch.from_numpy((rng.standard_normal(c) * 0.1).astype(np.float32)).cuda()
    rm = torch.from_numpy((rng.standard_normal(c) * 0.1).astype(np.float32)).cuda()
    rv = torch.from_numpy(rng.uniform(0.5, 2.0, c).astype(np.float32)).cuda()
    return x, g, b, rm, rv


def test_shapes_beyond_the_static_array_are_rejected():
    L = K.lib()
    cap = L.nblahip_bn_fwd_train_static_max_workspace()
    assert cap == 4 << 20
    # 2-D input with a million channels: the per-channel parameters alone need
    # 16 MB; rejected from the sizes, before any pointer or the device is used.
    assert L.nblahip_bn_workspace_bytes(4, 1 << 20, 1, 0) > cap
    code = L.nblahip_bn_fwd_train_static(None, None, None, None, None, None, None, None,
                                         4, 1 << 20, 1, 0.9, 1e-5, 0, None)
    assert code == -2
    assert b"workspace" in L.nblahip_error_string(code)


@pytest.mark.gpu
@pytest.mark.parametrize("pair,partials,knobs", CASES,
                         ids=["channel_last_f16", "planes_f32", "channel_last_on_chip_f16"])
def test_static_scratch_matches_the_workspace_entry_point(pair, partials, knobs):
    K.tune_reset()
    for name, value in knobs.items():
        K.tune_set(name, value)
    try:
        _static_against_workspace(pair, partials)
    finally:
        K.tune_reset()


def _static_against_workspace(pair, partials):
    import torch
    from oracle import norm_ref as R
    L = K.lib()
    for i, (shape, axis, dt) in enumerate(pair):
        print("case", shape, axis, dt, flush=True)
        x, g, b, rm, rv = _inputs(shape, axis, dt, seed=10 + i)
        s0, c, s2 = K._bn_sizes(x.shape, axis)
        assert 0 < L.nblahip_bn_workspace_bytes(s0, c, s2, K._dtype_code(x)) <= (4 << 20)
        rm_a, rv_a = rm.clone(), rv.clone()
        rm_b, rv_b = rm.clone(), rv.clone()
        # reference run first, with a profile of its kernels: the case must be
        # one that goes through the partials in the workspace
        K.check(L.nblahip_profile_enable(64))
        y_a, m_a, v_a = K.bn_forward_batch(x, b, g, rm_a, rv_a, axis, 0.9, 1e-5)
        torch.cuda.synchronize()
        _, fin = K.profile_query("bn_finalize_fwd_kernel")
        K.check(L.nblahip_profile_enable(0))
        assert fin == (1 if partials else 0), "the split reduction was expected / not expected"
        out = (torch.full_like(x, float("nan")), torch.empty_like(m_a), torch.empty_like(v_a))
        # (torch's allocator only sees the wrapper; the library itself never
        # calls an allocating routine)
        count = lambda: torch.cuda.memory_stats().get("allocation.all.allocated", 0)
        before = count()
        y_b, m_b, v_b = K.bn_forward_batch_static(x, b, g, rm_b, rv_b, axis, 0.9, 1e-5, out=out)
        assert count() == before
        torch.cuda.synchronize()
        for name, p, q in (("y", y_a, y_b), ("mean", m_a, m_b), ("var", v_a, v_b),
                           ("running mean", rm_a, rm_b), ("running var", rv_a, rv_b)):
            assert torch.equal(p, q), f"{name} differs from nblahip_bn_fwd_train on {shape}"
        xr = x.float().cpu().numpy().astype(np.float64)
        y_r, m_r, v_r, rm_r, rv_r = R.bn_forward_batch(
            xr, to_np(b), to_np(g), to_np(rm), to_np(rv), axis, 0.9, 1e-5)
        assert_close(to_np(y_b), y_r, dt, "y", "y vs oracle")
        assert_close(to_np(m_b), m_r, dt, "stat", "mean vs oracle")
        assert_close(to_np(v_b), v_r, dt, "stat", "var vs oracle")
        assert_close(to_np(rv_b), rv_r, dt, "stat", "running var vs oracle")


@pytest.mark.gpu
def test_empty_tensor_call_is_the_set_up_step():
    L = K.lib()
    assert L.nblahip_bn_fwd_train_static(None, None, None, None, None, None, None, None,
                                         0, 8, 4, 0.9, 1e-5, 0, None) == 0
