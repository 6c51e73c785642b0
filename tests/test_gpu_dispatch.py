"""Which kernel family each benchmark configuration (and a few shapes that sit
next to a plan boundary) dispatches to.  The chain of plans in the launch layer
is ordered by hand; a reordering that silently moved a configuration to another
family would change what the parity and in-place tests of that family cover.
The kernels that ran are read back from the library's per-kernel timing."""
import pytest
import torch

from _util import load_package

pytestmark = pytest.mark.gpu
K = load_package()
F32, F16 = torch.float32, torch.float16


@pytest.fixture(autouse=True)
def _default_knobs():
    K.tune_reset()
    yield
    K.tune_reset()
    K.check(K.lib().nblahip_profile_enable(0))


def kernels_of(fn):
    K.check(K.lib().nblahip_profile_enable(64))
    out = fn()
    torch.cuda.synchronize()
    names = K.profile_kernels()
    K.check(K.lib().nblahip_profile_enable(0))
    return out, names


def bn(shape, axis, dtype):
    c = shape[axis]
    x = torch.randn(shape, device="cuda").to(dtype)
    dy = torch.randn(shape, device="cuda").to(dtype)
    g, b = torch.ones(c, device="cuda"), torch.zeros(c, device="cuda")
    rm, rv = torch.zeros(c, device="cuda"), torch.ones(c, device="cuda")
    (y, m, v), f = kernels_of(lambda: K.bn_forward_batch(x, b, g, rm, rv, axis, 0.9, 1e-5))
    _, bw = kernels_of(lambda: K.bn_backward(x, dy, g, m, v, axis, 1e-5))
    return f, bw


def ln(rows, r, dtype):
    x = torch.randn(rows, r, device="cuda").to(dtype)
    dy = torch.randn(rows, r, device="cuda").to(dtype)
    g, b = torch.ones(r, device="cuda"), torch.zeros(r, device="cuda")
    (y, m, v), f = kernels_of(lambda: K.ln_forward(x, b, g, rows, 1e-5))
    _, bw = kernels_of(lambda: K.ln_backward(x, dy, g, m, v, rows, 1e-5))
    return f, bw


def gn(shape, groups, dtype, cl=False):
    c = shape[-1] if cl else shape[1]
    x = torch.randn(shape, device="cuda").to(dtype)
    dy = torch.randn(shape, device="cuda").to(dtype)
    g, b = torch.ones(c, device="cuda"), torch.zeros(c, device="cuda")
    if groups is None:
        (y, m, v), f = kernels_of(lambda: K.in_forward(x, b, g, 1e-5, channel_last=cl))
        _, bw = kernels_of(lambda: K.in_backward(x, dy, g, m, v, 1e-5, channel_last=cl))
    else:
        (y, m, v), f = kernels_of(lambda: K.gn_forward(x, b, g, groups, 1e-5, channel_last=cl))
        _, bw = kernels_of(lambda: K.gn_backward(x, dy, g, m, v, groups, 1e-5, channel_last=cl))
    return f, bw


# (id, runner, arguments, forward kernels, backward kernels)
TABLE = [
    # the five benchmark configurations
    ("C2", bn, ((32, 256, 56, 56), 1, F32), ["bn_onchip_fwd_kernel"], ["bn_onchip_bwd_kernel"]),
    ("C3_f32", ln, (16384, 1024, F32), ["row_fwd_kernel"], ["row_bwd_kernel_ln", "ln_param_reduce_kernel"]),
    ("C3_f16", ln, (16384, 1024, F16), ["row_fwd_kernel"], ["row_bwd_kernel_ln", "ln_param_reduce_kernel"]),
    ("C4_gn", gn, ((16, 256, 64, 64), 32, F16), ["row_fwd_kernel"], ["row_bwd_kernel_gn", "pair_param_reduce_kernel"]),
    ("C4_in", gn, ((16, 256, 64, 64), None, F16), ["row_fwd_kernel"], ["row_bwd_kernel_inc"]),
    ("C4_gn_nhwc", gn, ((16, 64, 64, 256), 32, F16, True), ["cl_split_fwd_kernel"],
     ["cl_split_bwd_kernel", "pair_param_reduce_cl_kernel"]),
    ("C4_in_nhwc", gn, ((16, 64, 64, 256), None, F16, True), ["cl_split_fwd_kernel"],
     ["cl_split_bwd_kernel", "pair_param_reduce_cl_kernel"]),
    ("C5", bn, ((256, 56, 56, 64), 3, F16), ["bn_cl_grid_fwd_kernel"], ["bn_cl_grid_bwd_kernel"]),
    # the shapes of the in-place cases, out of place
    ("chan_split", bn, ((37, 64, 32, 32), 1, F32), ["bn_chan_split_fwd_kernel"], ["bn_chan_split_bwd_kernel"]),
    ("rows_bn", bn, ((8, 64, 12, 12), 1, F32), ["row_fwd_kernel_bn"], ["row_bwd_kernel_bn"]),
    ("split_reduction", bn, ((8, 12, 14, 14), 1, F32), None, None),
    ("cl_cached", bn, ((8, 7, 7, 256), 3, F16), ["in_cl_row_fwd_kernel"], ["in_cl_row_bwd_kernel"]),
    ("tile", gn, ((2, 32, 32, 320), 32, F16, True), ["gn_cl_tile_fwd_kernel"],
     ["gn_cl_tile_bwd_kernel", "pair_param_reduce_cl_kernel"]),
]


@pytest.mark.parametrize("case", TABLE, ids=[t[0] for t in TABLE])
def test_family_of_each_configuration(case):
    _, run, args, fwd, bwd = case
    f, b = run(*args)
    if fwd is None:
        # the small split-reduction shape: whichever single-launch family takes
        # it, it is not one that exchanges between blocks
        assert not any("chan_split" in n or "grid" in n or "cl_split" in n for n in f + b), (f, b)
        return
    assert f == fwd, f
    assert b == bwd, b
