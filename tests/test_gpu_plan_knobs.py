"""Every plan a knob can switch on is held to the oracle.

A shape is served by one of several kernel families, chosen per call from the
plan knobs (NBLAHIP_<NAME> in the environment, or nblahip_tune_set).  The
default choice is what the other test files exercise; here each knob that
selects another kernel, or another grid for the same kernel, is set through
nblahip_tune_set, the forward and backward of a shape that the knob affects
run through the C-ABI, the results are compared with the float64 oracle, and
the kernels that ran (read back from the library's per-kernel timing) are
compared with the kernels of the default plan."""
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
def _default_knobs_afterwards():
    K.tune_reset()
    yield
    K.tune_reset()
    K.check(K.lib().nblahip_profile_enable(0))


# --------------------------------------------------------------- runners
# Each runs forward + backward on the device, checks every output against the
# oracle and returns nothing; inputs are seeded per case.
def run_bn(shape, axis, dtype, seed=1):
    dn = dtype_name(dtype)
    rng = np.random.default_rng(seed)
    c = shape[axis]
    x = rounded(rng.standard_normal(shape) * 2 + 1, dtype)
    dy = rounded(rng.standard_normal(shape), dtype)
    g, b = f32(rng.uniform(0.5, 1.5, c)), f32(rng.standard_normal(c) * 0.1)
    rm, rv = f32(rng.standard_normal(c) * 0.1), f32(rng.uniform(0.5, 2.0, c))
    y_r, m_r, v_r, rm_r, rv_r = R.bn_forward_batch(x, b, g, rm, rv, axis, 0.9, 1e-5)
    dx_r, dg_r, db_r = R.bn_backward_batch(x, dy, g, m_r, v_r, axis, 1e-5)
    xd, dyd, gd, bd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(b)
    rmd, rvd = to_dev(rm), to_dev(rv)
    y, m, v = K.bn_forward_batch(xd, bd, gd, rmd, rvd, axis, 0.9, 1e-5)
    assert_close(to_np(y), y_r, dn, "y", "y")
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(rmd), rm_r, dn, "stat", "running mean")
    assert_close(to_np(rvd), rv_r, dn, "stat", "running var")
    dx, dg, db = K.bn_backward(xd, dyd, gd, m, v, axis, 1e-5)
    assert_close(to_np(dx), dx_r, dn, "grad", "dx")
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


def run_bn_infer_bwd(shape, axis, dtype, seed=5):
    """Inference-mode backward (running statistics): dx alone, then dx, dgamma, dbeta."""
    dn = dtype_name(dtype)
    rng = np.random.default_rng(seed)
    c = shape[axis]
    x = rounded(rng.standard_normal(shape) * 2 + 1, dtype)
    dy = rounded(rng.standard_normal(shape), dtype)
    g = f32(rng.uniform(0.5, 1.5, c))
    rm, rv = f32(rng.standard_normal(c) * 0.1), f32(rng.uniform(0.5, 2.0, c))
    dx_r, dg_r, db_r = R.bn_backward_global(x, dy, g, rm, rv, axis, 1e-5)
    xd, dyd, gd, rmd, rvd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(rm), to_dev(rv)
    dx, _, _ = K.bn_backward(xd, dyd, gd, rmd, rvd, axis, 1e-5, batch_stat=False, need=(True, False, False))
    assert_close(to_np(dx), dx_r, dn, "grad", "dx alone")
    dx, dg, db = K.bn_backward(xd, dyd, gd, rmd, rvd, axis, 1e-5, batch_stat=False)
    assert_close(to_np(dx), dx_r, dn, "grad", "dx")
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


def run_ln(outer, Rr, dtype, seed=2):
    dn = dtype_name(dtype)
    rng = np.random.default_rng(seed)
    x = rounded(rng.standard_normal((outer, Rr)) + rng.uniform(-3, 3, (outer, 1)), dtype)
    dy = rounded(rng.standard_normal((outer, Rr)), dtype)
    g, b = f32(rng.standard_normal(Rr) * 0.1 + 1), f32(rng.standard_normal(Rr) * 0.1)
    y_r, m_r, v_r = R.ln_forward(x, b, g, outer, 1e-5)
    dx_r, dg_r, db_r = R.ln_backward(x, dy, g, m_r, v_r, outer, 1e-5)
    xd, dyd, gd, bd = to_dev(x, dtype), to_dev(dy, dtype), to_dev(g), to_dev(b)
    y, m, v = K.ln_forward(xd, bd, gd, outer, 1e-5)
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(y), y_r, dn, "y", "y")
    dx, dg, db = K.ln_backward(xd, dyd, gd, m, v, outer, 1e-5)
    assert_close(to_np(dx), dx_r, dn, "grad", "dx")
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


def _nc_inputs(n, c, sp, dtype, seed, channel_last):
    """Channel-first float64 views of the inputs (for the oracle) and the
    arrays in the caller's layout (for the device)."""
    rng = np.random.default_rng(seed)
    shape = (n, c) + tuple(sp)
    x = rounded(rng.standard_normal(shape) * 1.5 + rng.uniform(-2, 2, (n, c) + (1,) * len(sp)), dtype)
    dy = rounded(rng.standard_normal(shape), dtype)
    g, b = f32(rng.uniform(0.5, 1.5, c)), f32(rng.standard_normal(c) * 0.1)
    lay = (lambda a: np.ascontiguousarray(np.moveaxis(a, 1, -1))) if channel_last else (lambda a: a)
    return x, dy, g, b, lay


def run_gn(n, c, sp, groups, dtype, channel_last=False, seed=3):
    dn = dtype_name(dtype)
    x, dy, g, b, lay = _nc_inputs(n, c, sp, dtype, seed, channel_last)
    y_r, m_r, v_r = R.gn_forward(x, b, g, n, c, groups, 1e-5)
    dx_r, dg_r, db_r = R.gn_backward(x, dy, g, m_r, v_r, n, c, groups, 1e-5)
    xd, dyd, gd, bd = to_dev(lay(x), dtype), to_dev(lay(dy), dtype), to_dev(g), to_dev(b)
    y, m, v = K.gn_forward(xd, bd, gd, groups, 1e-5, channel_last=channel_last)
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(y), lay(y_r.reshape(x.shape)), dn, "y", "y")
    dx, dg, db = K.gn_backward(xd, dyd, gd, m, v, groups, 1e-5, channel_last=channel_last)
    assert_close(to_np(dx), lay(dx_r.reshape(x.shape)), dn, "grad", "dx")
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


def run_in(n, c, sp, dtype, channel_last=False, seed=4):
    dn = dtype_name(dtype)
    x, dy, g, b, lay = _nc_inputs(n, c, sp, dtype, seed, channel_last)
    y_r, m_r, v_r = R.in_forward(x, b, g, n, c, 1e-5)
    dx_r, dg_r, db_r = R.in_backward(x, dy, g, m_r, v_r, n, c, 1e-5)
    xd, dyd, gd, bd = to_dev(lay(x), dtype), to_dev(lay(dy), dtype), to_dev(g), to_dev(b)
    y, m, v = K.in_forward(xd, bd, gd, 1e-5, channel_last=channel_last)
    assert_close(to_np(m), m_r, dn, "stat", "mean")
    assert_close(to_np(v), v_r, dn, "stat", "var")
    assert_close(to_np(y), lay(y_r.reshape(x.shape)), dn, "y", "y")
    dx, dg, db = K.in_backward(xd, dyd, gd, m, v, 1e-5, channel_last=channel_last)
    assert_close(to_np(dx), lay(dx_r.reshape(x.shape)), dn, "grad", "dx")
    assert_close(to_np(dg), dg_r, dn, "pgrad", "dgamma")
    assert_close(to_np(db), db_r, dn, "pgrad", "dbeta")


# GroupNormalization rows about the channel-last kernels that own whole groups
# run with the split kernels (which take those shapes by default) switched off.
NO_SPLIT = {"GN_CL_SPLIT": 0}
# BatchNormalization rows about the kernels that give a channel one block run
# with the channel split over several blocks (the default for few channels) off.
NO_CHAN_SPLIT = {"BN_CHAN_SPLIT": 0}


def kernels_of(run, args, knobs):
    """Runs `run(*args)` (with its oracle checks) under `knobs`; returns the
    names of the kernels the library launched."""
    K.tune_reset()
    for name, value in knobs.items():
        K.tune_set(name, value)
    K.check(K.lib().nblahip_profile_enable(256))
    run(*args)
    torch.cuda.synchronize()
    names = K.profile_kernels()
    K.check(K.lib().nblahip_profile_enable(0))
    K.tune_reset()
    return names


# --------------------------------------------------------------- the table
# (id, runner, arguments, knobs, kernels the knob must bring in, kernels of the
# default plan that it must keep out).  The default plan of every row is run
# as well (same oracle checks) and must contain the "out" kernels: that pins
# that the shape is one the knob decides about.
SWITCHES = [
    # BatchNormalization, planes layout
    ("bn_onchip_off", run_bn, ((32, 64, 56, 56), 1, F16), {"BN_ONCHIP": 0},
     ["bn_stats_planes_kernel", "bn_apply_planes_kernel", "bn_bwd_reduce_planes_kernel",
      "bn_bwd_apply_planes_kernel"],
     ["bn_onchip_fwd_kernel", "bn_onchip_bwd_kernel"], NO_CHAN_SPLIT),
    ("bn_onchip_fwd_max", run_bn, ((32, 32, 56, 56), 1, F32), {"BN_ONCHIP_FWD_MAX": 16},
     ["bn_stats_planes_kernel"], ["bn_onchip_fwd_kernel"], NO_CHAN_SPLIT),
    ("bn_onchip_bwd_max", run_bn, ((32, 64, 56, 56), 1, F16), {"BN_ONCHIP_BWD_MAX": 8},
     ["bn_onchip_fwd_kernel", "bn_bwd_reduce_planes_kernel"], ["bn_onchip_bwd_kernel"], NO_CHAN_SPLIT),
    ("bn_onchip_min_pct_up", run_bn, ((32, 64, 56, 56), 1, F16),
     {"BN_ONCHIP_FWD_MIN_PCT": 100, "BN_ONCHIP_BWD_MIN_PCT": 100},
     ["bn_stats_planes_kernel", "bn_bwd_reduce_planes_kernel"],
     ["bn_onchip_fwd_kernel", "bn_onchip_bwd_kernel"], NO_CHAN_SPLIT),
    ("bn_chan_split_off", run_bn, ((32, 64, 56, 56), 1, F16), {"BN_CHAN_SPLIT": 0},
     ["bn_onchip_fwd_kernel", "bn_onchip_bwd_kernel"],
     ["bn_chan_split_fwd_kernel", "bn_chan_split_bwd_kernel"]),
    ("bn_rows_off", run_bn, ((32, 64, 14, 14), 1, F16), {"BN_ROWS": 0, "BN_MASKED_ONCHIP": 0},
     ["bn_stats_planes_kernel", "bn_finalize_fwd_kernel", "bn_apply_planes_kernel",
      "bn_finalize_bwd_kernel"], ["row_fwd_kernel_bn", "row_bwd_kernel_bn"]),
    ("bn_pack_off", run_bn, ((96, 384, 7, 7), 1, F16), {"BN_PACK": 0, "BN_MASKED_ONCHIP": 0},
     ["bn_stats_planes_kernel", "bn_bwd_reduce_planes_kernel"], ["bn_pack_fwd_kernel", "bn_pack_bwd_kernel"]),
    ("bn_pack_min_pct_up", run_bn, ((96, 384, 7, 7), 1, F16), {"BN_PACK_MIN_PCT": 50, "BN_MASKED_ONCHIP": 0},
     ["bn_stats_planes_kernel"], ["bn_pack_fwd_kernel", "bn_pack_bwd_kernel"]),
    ("bn_cl_grid_off", run_bn, ((100352, 64), 1, F16), {"BN_CL_GRID": 0},
     ["bn_stats_cl_kernel", "bn_finalize_fwd_kernel", "bn_apply_cl_kernel"], ["bn_cl_grid_fwd_kernel"],
     {"BN_CL_GRID_MIN_SLOTS": 1}),
    ("bn_cl_grid_from_more_vectors", run_bn, ((100352, 64), 1, F16), {"BN_CL_GRID_MIN_SLOTS": 9},
     ["bn_stats_cl_kernel"], ["bn_cl_grid_fwd_kernel"]),
    ("bn_cl_grid_from_fewer_rows", run_bn, ((6272, 64), 1, F16), {"BN_CL_GRID_MIN_ROWS": 1},
     ["bn_cl_grid_fwd_kernel", "bn_cl_grid_bwd_kernel"], ["cl_split_fwd_kernel"]),
    ("bn_masked_onchip_off", run_bn, ((64, 160, 17, 17), 1, F16), {"BN_MASKED_ONCHIP": 0},
     ["bn_apply_planes_kernel"], ["bn_masked_fwd_kernel", "bn_masked_bwd_kernel"]),
    ("bn_masked_onchip_min_pct_up", run_bn, ((64, 160, 17, 17), 1, F32), {"BN_MASKED_ONCHIP_MIN_PCT": 80},
     ["bn_apply_planes_kernel"], ["bn_masked_fwd_kernel", "bn_masked_bwd_kernel"]),
    ("bn_cl_grid_wide_off", run_bn, ((256, 14, 14, 256), 3, F16), {"BN_CL_GRID_WIDE": 0},
     ["cl_split_fwd_kernel", "bn_bwd_reduce_cl_kernel"], ["bn_cl_grid_fwd_kernel", "bn_cl_grid_bwd_kernel"]),
    ("bn_cl_grid_wide_from_more_rows", run_bn, ((256, 14, 14, 256), 3, F32), {"BN_CL_GRID_WIDE_MIN_ROWS": 60000, "BN_CL_GRID_WIDE_MIN_KB": 1000000},
     ["bn_stats_cl_kernel", "bn_bwd_reduce_cl_kernel"], ["bn_cl_grid_fwd_kernel", "bn_cl_grid_bwd_kernel"]),
    ("bn_cl_grid_strips_off", run_bn, ((128, 14, 14, 1024), 3, F16), {"BN_CL_GRID_STRIPS": 0},
     ["bn_stats_cl_kernel", "bn_bwd_reduce_cl_kernel"], ["bn_cl_grid_fwd_kernel", "bn_cl_grid_bwd_kernel"]),
    ("bn_cl_grid_strips_of_8_vectors", run_bn, ((256, 14, 14, 768), 3, F16), {"BN_CL_GRID_STRIP_VECS": 8},
     ["bn_cl_grid_fwd_kernel", "bn_cl_grid_bwd_kernel"], []),
    ("bn_cl_grid_strips_no_narrower_than", run_bn, ((256, 28, 28, 192), 3, F16), {"BN_CL_GRID_STRIP_MIN_VECS": 16},
     ["bn_stats_cl_kernel", "bn_bwd_reduce_cl_kernel"], ["bn_cl_grid_fwd_kernel", "bn_cl_grid_bwd_kernel"]),
    ("bn_cl_grid_wide_from_more_bytes", run_bn, ((64, 14, 14, 1024), 3, F32),
     {"BN_CL_GRID_WIDE_MIN_KB": 1000000, "BN_CL_GRID_WIDE_MIN_ROWS": 999999},
     ["cl_split_fwd_kernel", "cl_split_bwd_kernel"], ["bn_cl_grid_fwd_kernel", "bn_cl_grid_bwd_kernel"]),
    # (16 blocks instead of one per CU: 47 vectors per thread, the remainder streamed)
    ("bn_cl_grid_fewer_blocks", run_bn, ((48000, 128), 1, F16), {"BN_CL_GRID_BLOCKS": 16},
     ["bn_cl_grid_fwd_kernel", "bn_cl_grid_bwd_kernel"], []),
    ("bn_cl_grid_fwd_max_slots", run_bn, ((48000, 128), 1, F16), {"BN_CL_GRID_FWD_MAX_SLOTS": 25},
     ["bn_cl_grid_bwd_kernel"], ["bn_cl_grid_fwd_kernel"], {"BN_CL_GRID_BLOCKS": 16}),
    ("bn_cl_grid_bwd_max_slots", run_bn, ((48000, 128), 1, F16), {"BN_CL_GRID_BWD_MAX_SLOTS": 25},
     ["bn_cl_grid_fwd_kernel"], ["bn_cl_grid_bwd_kernel"], {"BN_CL_GRID_BLOCKS": 16}),
    ("bn_cl_grid_bwd_off", run_bn, ((100352, 64), 1, F16), {"BN_CL_GRID_BWD": 0},
     ["bn_cl_grid_fwd_kernel", "bn_bwd_reduce_cl_kernel", "bn_bwd_apply_cl_kernel"],
     ["bn_cl_grid_bwd_kernel"], {"BN_CL_GRID_MIN_SLOTS": 1}),
    ("bn_cl_cached_more_rows", run_bn, ((1568, 512), 1, F16), {"BN_CL_CACHED_MAX_ROWS": 2048},
     ["in_cl_row_fwd_kernel", "in_cl_row_bwd_kernel"], ["cl_split_fwd_kernel"]),
    ("bn_cl_cached_more_bytes", run_bn, ((1024, 4096), 1, F16), {"BN_CL_CACHED_MAX_KB": 16384},
     ["in_cl_row_fwd_kernel", "in_cl_row_bwd_kernel"], ["cl_split_fwd_kernel"]),
    ("bn_cl_cached_off", run_bn, ((32, 7, 7, 256), 3, F16), {"BN_CL_CACHED": 0},
     ["bn_stats_cl_kernel", "bn_apply_cl_kernel", "bn_bwd_reduce_cl_kernel", "bn_bwd_apply_cl_kernel"],
     ["in_cl_row_fwd_kernel", "in_cl_row_bwd_kernel"], {"BN_CL_SPLIT": 0}),
    ("bn_cl_split_off", run_bn, ((32, 14, 14, 256), 3, F16), {"BN_CL_SPLIT": 0},
     ["bn_stats_cl_kernel", "bn_apply_cl_kernel", "bn_bwd_reduce_cl_kernel", "bn_bwd_apply_cl_kernel"],
     ["cl_split_fwd_kernel", "cl_split_bwd_kernel"]),
    # rows: LayerNormalization / GroupNormalization / InstanceNormalization
    ("ln_force_stream", run_ln, (64, 1024, F32), {"FORCE_STREAM": 1},
     ["row_stats_stream_kernel", "row_apply_fwd_kernel", "ln_row_sums_stream_kernel",
      "row_bwd_dx_kernel", "ln_colgrad_stream_kernel"], ["row_fwd_kernel", "row_bwd_kernel_ln"]),
    ("gn_force_stream", run_gn, (4, 32, (16, 16), 8, F16), {"FORCE_STREAM": 1},
     ["row_stats_stream_kernel", "plane_sums_stream_kernel", "plane_to_row_factors_kernel"],
     ["row_fwd_kernel", "row_bwd_kernel_gn"]),
    ("in_force_stream", run_in, (4, 16, (32, 32), F32), {"FORCE_STREAM": 1},
     ["row_stats_stream_kernel", "plane_sums_stream_kernel"], ["row_fwd_kernel", "row_bwd_kernel_in"]),
    ("ln_long_rows_all_streaming", run_ln, (24, 18432, F16), {"LN_LONG_ROWS_CACHED": 0},
     ["ln_row_sums_stream_kernel", "row_bwd_dx_kernel"], ["row_bwd_kernel_lnx"]),
    # (the forward kernel has one name for every launch shape: these pin the results only)
    ("ln_fwd_block_per_row", run_ln, (1501, 4096, F16), {"LN_FWD_AHEAD": 0}, ["row_fwd_kernel"], []),
    ("ln_fwd_one_block_per_cu", run_ln, (1501, 4096, F16), {"LN_FWD_BLOCKS_PER_CU": 1}, ["row_fwd_kernel"], []),
    ("ln_no_three_vector_layouts", run_ln, (300, 6144, F16), {"ROW_NL3": 0}, ["row_fwd_kernel"], []),
    ("ln_bwd_no_rows_ahead", run_ln, (4100, 1024, F16), {"LN_BWD_AHEAD": 0}, ["row_bwd_kernel_ln"], []),
    ("ln_odd_rows_scalar", run_ln, (40, 1023, F16), {"LN_LOOSE": 0},
     ["row_bwd_kernel_ln"], ["ln_loose_bwd_kernel"]),
    ("in_rows_instead_of_channel_blocks", run_in, (4, 256, (32, 32), F16), {"IN_NO_CHANNEL_BLOCKS": 1},
     ["row_bwd_kernel_in", "pair_param_reduce_kernel"], ["row_bwd_kernel_inc"]),
    ("gn_float_groups_streamed", run_gn, (4, 64, (64, 64), 8, F32), {"GN_FLOAT_1024X8": 0},
     ["plane_sums_stream_kernel", "row_bwd_dx_kernel"], ["row_bwd_kernel_gn"]),
    ("gn_rows_onchip_off", run_gn, (4, 320, (64, 64), 32, F32), {"ROW_ONCHIP": 0},
     ["row_stats_stream_kernel", "row_apply_fwd_kernel"], ["row_onchip_fwd_kernel"]),
    ("in_rows_onchip_off", run_in, (2, 64, (256, 256), F32), {"ROW_ONCHIP": 0},
     ["row_stats_stream_kernel", "plane_sums_stream_kernel"],
     ["row_onchip_fwd_kernel", "bn_onchip_bwd_kernel"]),
    ("gn_onchip_bwd_off", run_gn, (4, 320, (64, 64), 32, F32), {"GN_ONCHIP_BWD": 0},
     ["plane_sums_stream_kernel", "row_bwd_dx_kernel"], ["gn_onchip_bwd_kernel"]),
    ("gn_onchip_bwd_from_more_vectors", run_gn, (4, 320, (64, 64), 32, F16), {"GN_ONCHIP_BWD_MIN_NL": 9},
     ["row_bwd_kernel_gn"], ["gn_onchip_bwd_kernel"]),
    ("gn_onchip_bwd_small_planes_off", run_gn, (4, 2560, (16, 16), 32, F16),
     {"GN_ONCHIP_BWD_SMALL_PLANES_MIN_NL": 99}, ["row_bwd_kernel_gn"], ["gn_onchip_bwd_kernel"]),
    ("rows_masked_groups_off", run_gn, (2, 64, (63, 63), 8, F16), {"ROW_MASKED_GROUPS": 0},
     ["row_stats_stream_kernel"], ["gn_planes_masked_fwd_kernel", "gn_planes_masked_bwd_kernel"]),
    ("rows_masked_groups_off_float", run_gn, (3, 12, (33, 33), 4, F32), {"ROW_MASKED": 0},
     [], ["gn_planes_masked_fwd_kernel", "gn_planes_masked_bwd_kernel"]),
    ("rows_masked_planes_off", run_gn, (2, 64, (63, 63), 8, F16), {"ROW_MASKED_PLANES": 0},
     ["gn_masked_fwd_kernel", "gn_masked_bwd_kernel"],
     ["gn_planes_masked_fwd_kernel", "gn_planes_masked_bwd_kernel"]),
    ("rows_masked_planes_off_float", run_gn, (2, 8, (65, 65), 2, F32), {"ROW_MASKED_PLANES": 0},
     ["gn_masked_fwd_kernel", "gn_masked_bwd_kernel"],
     ["gn_planes_masked_fwd_kernel", "gn_planes_masked_bwd_kernel"]),
    # (half planes of whole 8-byte vectors go to the plain row kernels: the knob brings the masked ones back)
    ("rows_masked_for_quad_planes", run_in, (6, 40, (14, 14), F16), {"ROW_MASKED_MID": 1},
     ["in_masked_fwd_kernel", "in_masked_bwd_kernel"], ["row_fwd_kernel"]),
    ("rows_masked_for_quad_planes_groups", run_gn, (6, 64, (14, 14), 8, F16), {"ROW_MASKED_MID": 1},
     ["gn_planes_masked_fwd_kernel", "gn_planes_masked_bwd_kernel"], ["row_fwd_kernel"]),
    ("rows_masked_off", run_in, (4, 32, (63, 63), F16), {"ROW_MASKED": 0},
     ["row_fwd_kernel"], ["in_masked_fwd_kernel", "in_masked_bwd_kernel"]),
    ("rows_masked_off_float", run_in, (3, 10, (9, 7), F32), {"ROW_MASKED": 0},
     ["row_fwd_kernel"], ["in_masked_fwd_kernel", "in_masked_bwd_kernel"]),
    ("rows_onchip_fwd_from_more_vectors", run_gn, (4, 320, (64, 64), 32, F16),
     {"ROW_ONCHIP_FWD_MIN_VECTORS": 8193}, ["row_fwd_kernel"], ["row_onchip_fwd_kernel"]),
    ("rows_onchip_min_pct_up", run_gn, (4, 320, (64, 64), 32, F32), {"ROW_ONCHIP_MIN_PCT": 100},
     ["row_stats_stream_kernel"], ["row_onchip_fwd_kernel"]),
    ("in_rows_onchip_bwd_min_pct_up", run_in, (2, 64, (256, 256), F32), {"ROW_ONCHIP_BWD_MIN_PCT": 100},
     ["row_onchip_fwd_kernel", "plane_sums_stream_kernel"], ["bn_onchip_bwd_kernel"]),
    # channel-last GroupNormalization / InstanceNormalization
    ("gn_cl_split_off", run_gn, (4, 1024, (32, 32), 128, F16, True), {"GN_CL_SPLIT": 0},
     ["gn_cl_wide_fwd_kernel", "cl_wide_bwd_kernel"], ["cl_split_fwd_kernel", "cl_split_bwd_kernel"]),
    ("gn_cl_split_off_float", run_gn, (2, 128, (20, 20), 8, F32, True), {"GN_CL_SPLIT": 0},
     ["gn_cl_row_fwd_kernel", "gn_cl_row_bwd_kernel"], ["cl_split_fwd_kernel", "cl_split_bwd_kernel"]),
    ("in_cl_split_off", run_in, (4, 1024, (32, 32), F16, True), {"GN_CL_SPLIT_INSTANCES": 0},
     ["in_cl_wide_fwd_kernel", "cl_wide_bwd_kernel"], ["cl_split_fwd_kernel", "cl_split_bwd_kernel"]),
    ("in_cl_split_off_float", run_in, (3, 64, (19, 19), F32, True), {"GN_CL_SPLIT_INSTANCES": 0},
     ["in_cl_row_fwd_kernel", "in_cl_row_bwd_kernel"], ["cl_split_fwd_kernel", "cl_split_bwd_kernel"]),
    ("gn_cl_tile_off", run_gn, (8, 320, (48, 48), 32, F16, True), {"GN_CL_TILE": 0},
     ["bn_stats_cl_kernel", "bn_bwd_reduce_cl_kernel"], ["gn_cl_tile_fwd_kernel", "gn_cl_tile_bwd_kernel"]),
    ("gn_cl_tile_off_float", run_gn, (8, 160, (33, 31), 16, F32, True), {"GN_CL_TILE": 0},
     ["bn_stats_cl_kernel", "bn_bwd_reduce_cl_kernel"], ["gn_cl_tile_fwd_kernel", "gn_cl_tile_bwd_kernel"]),
    ("gn_cl_tile_min_pct_up", run_gn, (4, 640, (40, 40), 32, F16, True), {"GN_CL_TILE_MIN_PCT": 60},
     ["bn_stats_cl_kernel", "bn_bwd_reduce_cl_kernel"], ["gn_cl_tile_fwd_kernel", "gn_cl_tile_bwd_kernel"]),
    ("gn_cl_wide_off", run_gn, (4, 1024, (32, 32), 128, F16, True),
     {"GN_CL_WIDE": 0, "GN_CL_WIDE_BWD": 0}, ["gn_cl_row_fwd_kernel", "gn_cl_row_bwd_kernel"],
     ["gn_cl_wide_fwd_kernel", "cl_wide_bwd_kernel"], NO_SPLIT),
    ("in_cl_wide_off", run_in, (4, 1024, (32, 32), F16, True),
     {"GN_CL_WIDE": 0, "GN_CL_WIDE_BWD": 0}, ["in_cl_row_fwd_kernel", "in_cl_row_bwd_kernel"],
     ["in_cl_wide_fwd_kernel", "cl_wide_bwd_kernel"], NO_SPLIT),
    ("gn_cl_cached_off", run_gn, (2, 128, (20, 20), 8, F32, True), {"GN_CL_CACHED": 0},
     ["bn_stats_cl_kernel", "gn_cl_finalize_fwd_kernel", "bn_bwd_reduce_cl_kernel",
      "gn_cl_finalize_bwd_kernel"], ["gn_cl_row_fwd_kernel", "gn_cl_row_bwd_kernel"],
     {**NO_SPLIT, "GN_CL_TILE": 0}),
    ("in_cl_cached_off", run_in, (2, 128, (20, 20), F32, True), {"IN_CL_CACHED": 0},
     ["bn_stats_cl_kernel", "gn_cl_finalize_fwd_kernel", "gn_cl_finalize_bwd_kernel"],
     ["in_cl_row_fwd_kernel", "in_cl_row_bwd_kernel"], NO_SPLIT),
    ("in_cl_min_positions_up", run_in, (4, 64, (8, 8), F16, True), {"IN_CL_MIN": 128},
     ["bn_stats_cl_kernel", "bn_bwd_reduce_cl_kernel"], ["in_cl_row_fwd_kernel", "in_cl_row_bwd_kernel"],
     NO_SPLIT),
]


@pytest.mark.parametrize("case", SWITCHES, ids=[c[0] for c in SWITCHES])
def test_plan_switch_changes_the_kernels_and_keeps_parity(case):
    _, run, args, knobs, must_run, must_not_run = case[:6]
    base = case[6] if len(case) > 6 else {}
    default = kernels_of(run, args, base)
    for name in must_not_run:
        assert name in default, f"default plan of {args} ran {default}, expected {name} among them"
    switched = kernels_of(run, args, {**base, **knobs})
    for name in must_run:
        assert name in switched, f"{knobs}: ran {switched}, expected {name}"
    for name in must_not_run:
        assert name not in switched, f"{knobs}: {name} still ran ({switched})"


# Knobs that keep the kernel names and change grids, thread maps, template
# instances or limits: parity under each value.  (id, runner, arguments, list
# of knob settings, kernels that must run, kernels that must not.)
GRIDS = [
    ("bn_blocks_per_cu", run_bn, ((16, 48, 28, 28), 1, F32),
     [{"BN_ROWS": 0, "BN_BLOCKS_PER_CU": v} for v in (1, 4, 64)],
     ["bn_stats_planes_kernel", "bn_finalize_fwd_kernel", "bn_finalize_bwd_kernel"], []),
    # channel-owning 1024-thread reduction blocks: no partials, no finalize kernel
    ("bn_direct_always", run_bn, ((16, 24, 28, 28), 1, F32), [{"BN_ROWS": 0, "BN_DIRECT": 1}],
     ["bn_stats_planes_kernel", "bn_bwd_reduce_planes_kernel"],
     ["bn_finalize_fwd_kernel", "bn_finalize_bwd_kernel"]),
    ("bn_direct_never", run_bn, ((8, 256, 28, 28), 1, F16), [{"BN_ROWS": 0, "BN_DIRECT": 0}],
     ["bn_stats_planes_kernel", "bn_finalize_fwd_kernel", "bn_finalize_bwd_kernel"], []),
    # (588 block steps of 1024 vectors: with one block per CU each block takes two or three)
    ("bn_apply_persistent", run_bn, ((64, 48, 28, 28), 1, F32),
     [{"BN_ROWS": 0, "BN_CHAN_SPLIT": 0, "BN_ONCHIP": 0, "BN_APPLY_BLOCKS_PER_CU": v} for v in (1, 3)],
     ["bn_apply_planes_kernel", "bn_bwd_apply_planes_kernel"], []),
    # (planes of 49 halves: vectors that straddle two planes, a table per block step)
    ("bn_apply_persistent_straddle", run_bn, ((256, 256, 7, 7), 1, F16),
     [{"BN_ROWS": 0, "BN_CHAN_SPLIT": 0, "BN_ONCHIP": 0, "BN_MASKED_ONCHIP": 0, "BN_PACK": 0,
       "BN_APPLY_BLOCKS_PER_CU": 1}],
     ["bn_stats_planes_kernel", "bn_apply_planes_kernel"], []),
    ("bn_masked_planes_off", run_bn, ((64, 64, 7, 7), 1, F16),
     [{"BN_ROWS": 0, "BN_MASKED_PLANES": 0, "BN_MASKED_ONCHIP": 0}],
     ["bn_stats_planes_kernel", "bn_apply_planes_kernel"], []),
    ("bn_cl_grids", run_bn, ((64, 28, 28, 64), 3, F16),
     [{"BN_CL_BLOCKS_PER_CU": a, "BN_CL_FWD_APPLY_BLOCKS_PER_CU": b, "BN_CL_APPLY_BLOCKS_PER_CU": c,
       "BN_CL_SPLIT": 0, "BN_CL_GRID": 0} for a, b, c in ((1, 1, 1), (2, 4, 2), (8, 3, 7))],
     ["bn_stats_cl_kernel", "bn_apply_cl_kernel", "bn_bwd_reduce_cl_kernel", "bn_bwd_apply_cl_kernel"],
     []),
    ("bn_cl_apply_tile", run_bn, ((16, 14, 14, 1000), 3, F16),
     [{"BN_CL_FWD_APPLY_TILE": t, "BN_CL_APPLY_TILE": u, "BN_CL_SPLIT": 0, "BN_CL_GRID": 0}
      for t, u in ((16, 256), (128, 16), (256, 128))],
     ["bn_stats_cl_kernel", "bn_apply_cl_kernel", "bn_bwd_reduce_cl_kernel", "bn_bwd_apply_cl_kernel"],
     []),
    ("bn_cl_grid_wide_fewer_rows", run_bn, ((128, 14, 14, 512), 3, F16), [{"BN_CL_GRID_WIDE_MIN_ROWS": 1}],
     ["bn_cl_grid_fwd_kernel", "bn_cl_grid_bwd_kernel"], []),
    ("bn_onchip_few_channels", run_bn, ((32, 4, 56, 56), 1, F16),
     [{"BN_ONCHIP_FWD_MIN_PCT": 1, "BN_ONCHIP_BWD_MIN_PCT": 1, **NO_CHAN_SPLIT}],
     ["bn_onchip_fwd_kernel", "bn_onchip_bwd_kernel"], []),
    # planes that share cache lines with their neighbours: ordinary stores there, or not
    ("bn_onchip_edge_stores_off", run_bn, ((256, 64, 14, 14), 1, F32),
     [{"BN_EDGE_STORES_MAX_BYTES": 0, **NO_CHAN_SPLIT}], ["bn_onchip_fwd_kernel", "bn_onchip_bwd_kernel"], []),
    ("bn_rows_edge_stores_off", run_bn, ((32, 64, 14, 14), 1, F16), [{"BN_EDGE_STORES_MAX_BYTES": 0}],
     ["row_fwd_kernel_bn", "row_bwd_kernel_bn"], []),
    ("bn_onchip_edge_stores_longer_planes", run_bn, ((128, 64, 28, 28), 1, F16),
     [{"BN_EDGE_STORES_MAX_BYTES": 4096}], ["bn_onchip_fwd_kernel", "bn_onchip_bwd_kernel"], []),
    ("bn_onchip_streamed_few_channels", run_bn, ((64, 8, 56, 56), 1, F32),
     [{"BN_ONCHIP_STREAMED_MIN_PCT": 1, **NO_CHAN_SPLIT}], ["bn_onchip_fwd_kernel", "bn_onchip_bwd_kernel"], []),
    # a channel split over 8 blocks on a quarter of the CUs; every partner's part
    # recomputed because no poll is allowed
    ("bn_chan_split_few_blocks", run_bn, ((40, 8, 32, 32), 1, F32), [{"BN_CHAN_SPLIT_MIN_PCT": 1}],
     ["bn_chan_split_fwd_kernel", "bn_chan_split_bwd_kernel"], []),
    ("bn_chan_split_no_polls", run_bn, ((32, 64, 56, 56), 1, F16), [{"XCHG_SPIN": 0}],
     ["bn_chan_split_fwd_kernel", "bn_chan_split_bwd_kernel"], []),
    ("bn_pack_few_channels", run_bn, ((48, 16, 7, 7), 1, F16), [{"BN_PACK_SHORT_MIN_PCT": 0}],
     ["bn_pack_fwd_kernel", "bn_pack_bwd_kernel"], []),
    ("bn_pack_plain_block_order", run_bn, ((96, 384, 7, 7), 1, F16),
     [{"BN_PACK_XCD_MAP": 0}, {"BN_PACK_EDGE_STORES": 0}],
     ["bn_pack_fwd_kernel", "bn_pack_bwd_kernel"], []),
    ("ln_bwd_blocks_per_cu", run_ln, (4096, 1024, F16), [{"LN_BWD_BLOCKS_PER_CU": v} for v in (1, 2, 4)],
     ["row_bwd_kernel_ln", "ln_param_reduce_kernel"], []),
    ("ln_wave_per_short_row", run_ln, (1000, 32, F32), [{"ROW_SUBWAVE": 0}],
     ["row_fwd_kernel", "row_bwd_kernel_ln"], []),
    ("ln_forced_subwave_layout", run_ln, (513, 128, F32), [{"ROW_TPR": 8, "ROW_NL": 4},
                                                           {"ROW_TPR": 16, "ROW_NL": 2}],
     ["row_fwd_kernel", "row_bwd_kernel_ln"], []),
    ("rows_onchip_few_rows", run_in, (1, 8, (256, 256), F32),
     [{"ROW_ONCHIP_MIN_PCT": 1, "ROW_ONCHIP_BWD_MIN_PCT": 1}],
     ["row_onchip_fwd_kernel", "bn_onchip_bwd_kernel"], []),
    ("rows_onchip_streamed_few_rows", run_in, (1, 8, (512, 512), F16),
     [{"ROW_ONCHIP_STREAMED_MIN_PCT": 1}], ["row_onchip_fwd_kernel", "bn_onchip_bwd_kernel"], []),
    # the split kernels: every block shape, and every partner's part recomputed
    # because no poll is allowed (what a block does when a partner is late)
    ("gn_cl_split_shapes", run_gn, (3, 128, (40, 40), 16, F16, True),
     [{"GN_CL_SPLIT_TPR": t, "GN_CL_SPLIT_NL": n} for t, n in ((256, 4), (256, 8), (512, 4), (512, 8),
                                                                (1024, 4), (1024, 8))],
     ["cl_split_fwd_kernel", "cl_split_bwd_kernel"], []),
    ("gn_cl_split_shapes_float", run_gn, (2, 64, (37, 37), 8, F32, True),
     [{"GN_CL_SPLIT_TPR": t, "GN_CL_SPLIT_NL": n} for t, n in ((256, 4), (256, 8), (512, 4), (512, 8),
                                                                (1024, 4), (1024, 8))],
     ["cl_split_fwd_kernel", "cl_split_bwd_kernel"], []),
    ("gn_cl_split_no_polls", run_gn, (3, 128, (40, 40), 16, F16, True), [{"XCHG_SPIN": 0}],
     ["cl_split_fwd_kernel", "cl_split_bwd_kernel"], []),
    ("in_cl_split_no_polls", run_in, (2, 64, (30, 30), F32, True), [{"XCHG_SPIN": 0}],
     ["cl_split_fwd_kernel", "cl_split_bwd_kernel"], []),
    ("gn_cl_tile_no_polls", run_gn, (8, 320, (48, 48), 32, F16, True), [{"XCHG_SPIN": 0}],
     ["gn_cl_tile_fwd_kernel", "gn_cl_tile_bwd_kernel"], []),
    ("gn_cl_tile_no_polls_float", run_gn, (8, 160, (33, 31), 16, F32, True), [{"XCHG_SPIN": 0}],
     ["gn_cl_tile_fwd_kernel", "gn_cl_tile_bwd_kernel"], []),
    ("gn_cl_tile_few_blocks", run_gn, (1, 320, (6, 6), 32, F16, True), [{"GN_CL_TILE_MIN_PCT": 0}],
     ["gn_cl_tile_fwd_kernel", "gn_cl_tile_bwd_kernel"], []),
    ("gn_cl_wide_plain_block_order", run_gn, (4, 1024, (32, 32), 128, F16, True),
     [{"GN_CL_XCD_MAP": 0, **NO_SPLIT}],
     ["gn_cl_wide_fwd_kernel", "cl_wide_bwd_kernel"], []),
    ("in_cl_wide_plain_block_order", run_in, (4, 1024, (32, 32), F16, True),
     [{"GN_CL_XCD_MAP": 0, **NO_SPLIT}],
     ["in_cl_wide_fwd_kernel", "cl_wide_bwd_kernel"], []),
    # four groups per block, 16 vectors per thread, on a quarter of the CUs
    ("gn_cl_wide_fewer_blocks", run_gn, (8, 256, (64, 64), 32, F16, True),
     [{"GN_CL_WIDE_MIN_PCT": 25, **NO_SPLIT}],
     ["gn_cl_wide_fwd_kernel"], []),
    ("gn_cl_rows_plain_block_order", run_gn, (2, 128, (20, 20), 8, F32, True),
     [{"GN_CL_XCD_MAP": 0, **NO_SPLIT}],
     ["gn_cl_row_fwd_kernel", "gn_cl_row_bwd_kernel"], []),
    ("in_cl_rows_plain_block_order", run_in, (2, 128, (20, 20), F16, True),
     [{"GN_CL_XCD_MAP": 0, "GN_CL_WIDE": 0, "GN_CL_WIDE_BWD": 0, **NO_SPLIT}],
     ["in_cl_row_fwd_kernel", "in_cl_row_bwd_kernel"], []),
    ("in_cl_fewer_positions", run_in, (4, 64, (4, 4), F16, True), [{"IN_CL_MIN": 8, **NO_SPLIT}],
     ["in_cl_row_fwd_kernel", "in_cl_row_bwd_kernel"], []),
    # the fold of the LayerNormalization column partials in 256-byte runs, from any size / never
    ("ln_param_reduce_wide", run_ln, (300, 2048, F16), [{"LN_REDUCE_WIDE_MIN_KB": 0}],
     ["row_bwd_kernel_ln", "ln_param_reduce_wide_kernel"], ["ln_param_reduce_kernel"]),
    ("ln_param_reduce_wide_float", run_ln, (77, 5124, F32), [{"LN_REDUCE_WIDE_MIN_KB": 0}],
     ["ln_param_reduce_wide_kernel"], ["ln_param_reduce_kernel"]),
    ("ln_param_reduce_narrow", run_ln, (2048, 8192, F16), [{"LN_REDUCE_WIDE_MIN_KB": 1000000}],
     ["row_bwd_kernel_ln", "ln_param_reduce_kernel"], ["ln_param_reduce_wide_kernel"]),
    # half rows of 257 - 512 vectors: 256 threads x 2 vectors with the next row ahead (default),
    # 512 x 1, and the layouts a sweep can force
    ("ln_bwd_256x2_off", run_ln, (2304, 3072, F16), [{"LN_BWD_256X2": 0}, {"LN_BWD_AHEAD": 0}],
     ["row_bwd_kernel_ln"], []),
    ("ln_bwd_forced_layouts", run_ln, (2100, 2560, F16),
     [{"LN_BWD_TPR": t, "LN_BWD_NL": n} for t, n in ((512, 1), (256, 2), (256, 3), (512, 2), (256, 4), (512, 4))],
     ["row_bwd_kernel_ln"], []),
    ("ln_bwd_forced_layouts_float", run_ln, (2100, 1000, F32),
     [{"LN_BWD_TPR": t, "LN_BWD_NL": n} for t, n in ((64, 4), (256, 1), (256, 2), (512, 1), (512, 3))],
     ["row_bwd_kernel_ln"], []),
    # channel-last rows that are no whole number of 128-byte segments: column strips of 64 bytes
    # on the grid-resident kernels (default where the chip holds the tensor), or the three launches
    ("bn_cl_grid_narrow_strips_off", run_bn, ((16, 28, 28, 96), 3, F16), [{"BN_CL_GRID_STRIP_MIN_VECS": 8}],
     ["bn_stats_cl_kernel", "bn_bwd_reduce_cl_kernel"], ["bn_cl_grid_fwd_kernel", "bn_cl_grid_bwd_kernel"]),
    ("bn_cl_grid_narrow_strips", run_bn, ((16, 28, 28, 96), 3, F16), [{}],
     ["bn_cl_grid_fwd_kernel", "bn_cl_grid_bwd_kernel"], []),
    ("bn_cl_grid_narrow_strips_float", run_bn, ((16, 28, 28, 80), 3, F32), [{}],
     ["bn_cl_grid_fwd_kernel", "bn_cl_grid_bwd_kernel"], []),
    # inference-mode backward: dx through the forward's inference apply over dy (default) / the backward apply
    ("bn_infer_bwd_as_apply", run_bn_infer_bwd, ((16, 48, 28, 28), 1, F16), [{}],
     ["bn_apply_planes_kernel", "bn_bwd_reduce_planes_kernel"], ["bn_bwd_apply_planes_kernel"]),
    ("bn_infer_bwd_as_apply_channel_last", run_bn_infer_bwd, ((16, 28, 28, 48), 3, F32), [{}],
     ["bn_apply_cl_kernel", "bn_bwd_reduce_cl_kernel"], ["bn_bwd_apply_cl_kernel"]),
    ("bn_infer_bwd_as_apply_odd_planes", run_bn_infer_bwd, ((16, 48, 13, 13), 1, F16), [{}],
     ["bn_apply_planes_kernel"], ["bn_bwd_apply_planes_kernel"]),
    ("bn_infer_bwd_through_backward_apply", run_bn_infer_bwd, ((16, 48, 28, 28), 1, F16),
     [{"BN_INFER_BWD_AS_APPLY": 0}], ["bn_bwd_apply_planes_kernel"], ["bn_apply_planes_kernel"]),
    # few channel packs where a block per channel holds the channel: the masked kernels (default) / packs
    ("bn_pack_few_packs_to_masked", run_bn, ((256, 96, 7, 7), 1, F16), [{}],
     ["bn_masked_fwd_kernel", "bn_masked_bwd_kernel"], ["bn_pack_fwd_kernel"]),
    ("bn_pack_few_packs", run_bn, ((256, 96, 7, 7), 1, F16), [{"BN_PACK_MIN_PCT_MASKED": 1}],
     ["bn_pack_fwd_kernel", "bn_pack_bwd_kernel"], ["bn_masked_fwd_kernel"]),
    ("bn_cl_grid_narrow_few_rows", run_bn, ((16, 14, 14, 96), 3, F16), [{}],
     ["bn_cl_grid_fwd_kernel", "bn_cl_grid_bwd_kernel"], []),
    ("bn_cl_grid_narrow_from_more_rows", run_bn, ((16, 14, 14, 96), 3, F16), [{"BN_CL_GRID_NARROW_MIN_ROWS": 10240}],
     ["bn_stats_cl_kernel", "bn_bwd_reduce_cl_kernel"], ["bn_cl_grid_fwd_kernel"]),
    ("bn_cl_grid_narrow_backward_limit", run_bn, ((16, 28, 28, 160), 3, F16),
     [{"BN_CL_GRID_NARROW_BWD_MAX_KB": 1024}], ["bn_cl_grid_fwd_kernel", "bn_bwd_reduce_cl_kernel"],
     ["bn_cl_grid_bwd_kernel"]),
    ("bn_cl_grid_narrow_backward_limit_float", run_bn, ((16, 28, 28, 80), 3, F32),
     [{"BN_CL_GRID_NARROW_BWD_MAX_KB_F32": 1024}], ["bn_cl_grid_fwd_kernel", "bn_bwd_reduce_cl_kernel"],
     ["bn_cl_grid_bwd_kernel"]),
    ("in_forced_wave_layouts", run_in, (6, 40, (32, 32), F16),
     [{"ROW_TPR": t, "ROW_NL": n} for t, n in ((64, 2), (64, 4), (256, 1), (256, 2), (512, 1), (1024, 1))],
     ["row_fwd_kernel"], []),
    # block order by line-sharing sets only where the sets divide a sample's units
    ("gn_cl_rows_block_order_whole_sets", run_gn, (2, 120, (20, 20), 15, F32, True),
     [{"GN_CL_XCD_MAP": m, **NO_SPLIT} for m in (1, 2)],
     ["gn_cl_row_fwd_kernel", "gn_cl_row_bwd_kernel"], []),
    # groups no split kernel takes, tensors beyond 4 MiB: the tile kernels ahead
    # of the cached ones from a number of vectors per group, either way round
    ("gn_cl_tile_first_half", run_gn, (16, 200, (28, 28), 25, F16, True),
     [{"GN_CL_TILE_FIRST_FWD": 0, "GN_CL_TILE_FIRST_BWD": 0}],
     ["gn_cl_tile_fwd_kernel", "gn_cl_tile_bwd_kernel"], []),
    ("gn_cl_tile_later_half", run_gn, (16, 200, (28, 28), 25, F16, True),
     [{"GN_CL_TILE_FIRST_FWD": 100000, "GN_CL_TILE_FIRST_BWD": 100000}],
     ["gn_cl_row_fwd_kernel", "gn_cl_row_bwd_kernel"], []),
    ("gn_cl_tile_first_float", run_gn, (32, 100, (24, 24), 25, F32, True),
     [{"GN_CL_TILE_FIRST_FWD_F32": 0, "GN_CL_TILE_FIRST_BWD_F32": 0}],
     ["gn_cl_tile_fwd_kernel", "gn_cl_tile_bwd_kernel"], []),
    ("gn_cl_tile_later_float", run_gn, (32, 100, (24, 24), 25, F32, True),
     [{"GN_CL_TILE_FIRST_FWD_F32": 100000, "GN_CL_TILE_FIRST_BWD_F32": 100000}],
     ["gn_cl_row_fwd_kernel", "gn_cl_row_bwd_kernel"], []),
    # InstanceNormalization proper beyond 4 MiB: most positions the cached kernels take
    ("in_cl_cached_more_positions", run_in, (8, 200, (48, 48), F16, True), [{"IN_CL_MAX": 4096}],
     ["in_cl_row_fwd_kernel"], []),
    ("in_cl_cached_fewer_positions", run_in, (16, 200, (40, 40), F16, True), [{"IN_CL_MAX": 1024}],
     ["bn_stats_cl_kernel", "bn_bwd_reduce_cl_kernel"], ["in_cl_row_fwd_kernel", "in_cl_row_bwd_kernel"]),
    ("in_cl_cached_positions_float", run_in, (32, 100, (28, 28), F32, True),
     [{"IN_CL_MAX_F32_FWD": 512, "IN_CL_MAX_F32_BWD": 1024}],
     ["bn_stats_cl_kernel", "in_cl_row_bwd_kernel"], ["in_cl_row_fwd_kernel", "bn_bwd_reduce_cl_kernel"]),
]


@pytest.mark.parametrize("case", GRIDS, ids=[c[0] for c in GRIDS])
def test_grid_and_limit_knobs_keep_parity(case):
    _, run, args, settings, expected, absent = case
    for knobs in settings:
        ran = kernels_of(run, args, knobs)
        for name in expected:
            assert name in ran, f"{knobs}: ran {ran}, expected {name}"
        for name in absent:
            assert name not in ran, f"{knobs}: {name} ran ({ran})"
