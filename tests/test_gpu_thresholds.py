"""Plan switches that depend on a tuned size or a share of the CUs: one shape
just below and one just above each threshold.  On both sides the default plan
is held to the oracle, so is the plan the other side of the threshold would
take (forced through the knob), the kernels that ran are read back to pin that
the knob decides about the shape, and the default plan must not be more than
15 % (+ 1 us) slower than the other one - a threshold that has drifted away
from the crossover shows up here instead of staying silent.  Times are sums of
the library's per-kernel event timing over forward + backward, averaged over
repetitions that walk rotated buffer sets.  The measured pairs are written to
thresholds.json in the directory that NBLAHIP_RESULTS_DIR names, if it is set."""
import json
import os

import pytest
import torch

from _util import load_package
import test_gpu_plan_knobs as P

pytestmark = pytest.mark.gpu
K = load_package()
F32, F16 = torch.float32, torch.float16
RESULTS = {}


@pytest.fixture(autouse=True)
def _default_knobs():
    K.tune_reset()
    yield
    K.tune_reset()
    K.check(K.lib().nblahip_profile_enable(0))


@pytest.fixture(scope="module", autouse=True)
def _dump():
    yield
    out = os.environ.get("NBLAHIP_RESULTS_DIR", "")
    if out and os.path.isdir(out) and RESULTS:
        with open(os.path.join(out, "thresholds.json"), "w") as f:
            json.dump(RESULTS, f, indent=1)


# ---------------------------------------------------------------- timing runners
def _sets(nbytes_per_set):
    return int(max(2, min(16, -(-(768 << 20) // max(1, nbytes_per_set)))))


def _time(calls, nsets, reps=12):
    """Microseconds of kernel time per call of calls(i) (i: buffer set), and the
    kernels that ran."""
    for i in range(nsets):
        calls(i)
    torch.cuda.synchronize()
    K.check(K.lib().nblahip_profile_enable(64 * reps))
    for r in range(reps):
        calls(r % nsets)
    torch.cuda.synchronize()
    names = K.profile_kernels()
    total = sum(K.profile_query(n)[0] for n in names)
    K.check(K.lib().nblahip_profile_enable(0))
    return total * 1e3 / reps, names


def time_bn(shape, axis, dtype):
    c = shape[axis]
    n = _sets(4 * torch.empty(shape, dtype=dtype).numel() * (2 if dtype == F16 else 4))
    xs = [torch.randn(shape, device="cuda").to(dtype) for _ in range(n)]
    dys = [torch.randn(shape, device="cuda").to(dtype) for _ in range(n)]
    g, b = torch.ones(c, device="cuda"), torch.zeros(c, device="cuda")
    rm, rv = torch.zeros(c, device="cuda"), torch.ones(c, device="cuda")

    def calls(i):
        y, m, v = K.bn_forward_batch(xs[i], b, g, rm, rv, axis, 0.9, 1e-5)
        K.bn_backward(xs[i], dys[i], g, m, v, axis, 1e-5)
    return _time(calls, n)


def time_gn(n_, c, sp, groups, dtype, channel_last=False):
    shape = (n_,) + tuple(sp) + (c,) if channel_last else (n_, c) + tuple(sp)
    n = _sets(4 * torch.empty(shape, dtype=dtype).numel() * (2 if dtype == F16 else 4))
    xs = [torch.randn(shape, device="cuda").to(dtype) for _ in range(n)]
    dys = [torch.randn(shape, device="cuda").to(dtype) for _ in range(n)]
    g, b = torch.ones(c, device="cuda"), torch.zeros(c, device="cuda")

    def calls(i):
        if groups is None:
            y, m, v = K.in_forward(xs[i], b, g, 1e-5, channel_last=channel_last)
            K.in_backward(xs[i], dys[i], g, m, v, 1e-5, channel_last=channel_last)
        else:
            y, m, v = K.gn_forward(xs[i], b, g, groups, 1e-5, channel_last=channel_last)
            K.gn_backward(xs[i], dys[i], g, m, v, groups, 1e-5, channel_last=channel_last)
    return _time(calls, n)


def time_in(n_, c, sp, dtype, channel_last=False):
    return time_gn(n_, c, sp, None, dtype, channel_last)


TIMERS = {P.run_bn: time_bn, P.run_gn: time_gn, P.run_in: time_in}

# (id, runner, base knobs, [(side, arguments, knobs that force the other side's
# plan, kernel that the default plan runs, kernel that the forced plan runs)])
NCS = P.NO_CHAN_SPLIT
CASES = [
    # a channel with a streamed remainder held on one CU: from channels for 37 % of the CUs
    ("bn_onchip_streamed_min_pct", P.run_bn, NCS,
     [("below", ((32, 64, 56, 56), 1, F32), {"BN_ONCHIP_STREAMED_MIN_PCT": 1}, "bn_bwd_reduce_planes_kernel", "bn_onchip_bwd_kernel"),
      ("above", ((32, 112, 56, 56), 1, F32), {"BN_ONCHIP_STREAMED_MIN_PCT": 100}, "bn_onchip_bwd_kernel", "bn_bwd_reduce_planes_kernel")]),
    # whole channels held on one CU: from the first channel (the old thresholds, an
    # eighth and a quarter of the CUs, left 20 - 45 % on the table below them)
    ("bn_onchip_whole_channels", P.run_bn, NCS,
     [("few", ((16, 8, 56, 56), 1, F32), {"BN_ONCHIP_FWD_MIN_PCT": 100, "BN_ONCHIP_BWD_MIN_PCT": 100}, "bn_onchip_bwd_kernel", "bn_bwd_reduce_planes_kernel"),
      ("more", ((32, 60, 56, 56), 1, F16), {"BN_ONCHIP_FWD_MIN_PCT": 100, "BN_ONCHIP_BWD_MIN_PCT": 100}, "bn_onchip_bwd_kernel", "bn_bwd_reduce_planes_kernel")]),
    # a channel split over up to 8 blocks: from the first channel
    ("bn_chan_split_min_pct", P.run_bn, {},
     [("few", ((32, 2, 56, 56), 1, F16), {"BN_CHAN_SPLIT_MIN_PCT": 100}, "bn_chan_split_fwd_kernel", None),
      ("more", ((32, 16, 56, 56), 1, F32), {"BN_CHAN_SPLIT_MIN_PCT": 100}, "bn_chan_split_fwd_kernel", None)]),
    # channel packs of 7 x 7 planes: from the first pack where the row kernels do not take the channel
    ("bn_pack_min_pct", P.run_bn, {"BN_MASKED_ONCHIP": 0},
     [("few", ((96, 240, 7, 7), 1, F16), {"BN_PACK_MIN_PCT": 100}, "bn_pack_fwd_kernel", "bn_stats_planes_kernel"),
      ("short_below", ((32, 256, 7, 7), 1, F16), {"BN_PACK_SHORT_MIN_PCT": 1}, "row_fwd_kernel_bn", "bn_pack_fwd_kernel"),
      ("short_below_more", ((32, 1024, 7, 7), 1, F16), {"BN_PACK_SHORT_MIN_PCT": 1}, "row_fwd_kernel_bn", "bn_pack_fwd_kernel"),
      ("short_above", ((64, 2048, 7, 7), 1, F16), {"BN_PACK_SHORT_MIN_PCT": 101}, "bn_pack_fwd_kernel", "row_fwd_kernel_bn")]),
    # ... long channels in few packs, where a block per channel holds the channel: packs from 16 % of the CUs
    ("bn_pack_min_pct_masked", P.run_bn, {},
     [("below", ((256, 256, 7, 7), 1, F16), {"BN_PACK_MIN_PCT_MASKED": 1}, "bn_masked_fwd_kernel", "bn_pack_fwd_kernel"),
      ("above", ((256, 512, 7, 7), 1, F16), {"BN_PACK_MIN_PCT_MASKED": 100}, "bn_pack_fwd_kernel", "bn_masked_fwd_kernel"),
      ("below_f32", ((128, 160, 7, 7), 1, F32), {"BN_PACK_MIN_PCT_MASKED": 1}, "bn_masked_fwd_kernel", "bn_pack_fwd_kernel")]),
    # odd planes with a channel held by one block: from the first channel
    ("bn_masked_onchip_min_pct", P.run_bn, {},
     [("few", ((64, 8, 17, 17), 1, F16), {"BN_MASKED_ONCHIP_MIN_PCT": 100}, "bn_masked_fwd_kernel", None),
      ("more", ((64, 32, 17, 17), 1, F32), {"BN_MASKED_ONCHIP_MIN_PCT": 100}, "bn_masked_fwd_kernel", None)]),
    # channel-last, the tensor held on the chip: from 10240 rows
    ("bn_cl_grid_min_rows", P.run_bn, {},
     [("below", ((6272, 64), 1, F16), {"BN_CL_GRID_MIN_ROWS": 1}, "cl_split_fwd_kernel", "bn_cl_grid_fwd_kernel"),
      ("above", ((12544, 64), 1, F16), {"BN_CL_GRID_MIN_ROWS": 999999}, "bn_cl_grid_fwd_kernel", "cl_split_fwd_kernel"),
      ("above_f32", ((12544, 128), 1, F32), {"BN_CL_GRID_MIN_ROWS": 999999}, "bn_cl_grid_fwd_kernel", "cl_split_fwd_kernel")]),
    # ... with more than 128 channels: from 10240 rows as well
    ("bn_cl_grid_wide_min_rows", P.run_bn, {},
     [("below", ((32, 14, 14, 256), 3, F16), {"BN_CL_GRID_WIDE_MIN_ROWS": 1}, "cl_split_fwd_kernel",
       "bn_cl_grid_fwd_kernel"),
      ("above", ((64, 14, 14, 256), 3, F16), {"BN_CL_GRID_WIDE_MIN_ROWS": 999999, "BN_CL_GRID_WIDE_MIN_KB": 1000000},
       "bn_cl_grid_fwd_kernel", "cl_split_fwd_kernel")]),
    # ... or from 24 MiB
    ("bn_cl_grid_wide_min_kb", P.run_bn, {},
     [("below", ((32, 14, 14, 1024), 3, F16), {"BN_CL_GRID_WIDE_MIN_KB": 1}, "cl_split_fwd_kernel", "bn_cl_grid_fwd_kernel"),
      ("above", ((128, 7, 7, 2048), 3, F16), {"BN_CL_GRID_WIDE_MIN_KB": 1000000}, "bn_cl_grid_fwd_kernel",
       "cl_split_fwd_kernel")]),
    # few rows, a block per channel vector: up to 1024 rows and 4 MiB
    ("bn_cl_cached_max", P.run_bn, {},
     [("below", ((1024, 1024), 1, F16), {"BN_CL_CACHED": 0}, "in_cl_row_fwd_kernel", "cl_split_fwd_kernel"),
      ("above_rows", ((1568, 2048), 1, F16), {"BN_CL_CACHED_MAX_ROWS": 4096, "BN_CL_CACHED_MAX_KB": 1000000},
       "cl_split_fwd_kernel", "in_cl_row_fwd_kernel"),
      ("above_bytes", ((1024, 4096), 1, F16), {"BN_CL_CACHED_MAX_KB": 1000000}, "cl_split_fwd_kernel",
       "in_cl_row_fwd_kernel")]),
    # ... and up to 80 / 50 vectors per thread (25 / 21 held): beyond, three launches are as fast
    ("bn_cl_grid_max_slots", P.run_bn, {},
     [("below", ((256, 28, 28, 512), 3, F16), {"BN_CL_GRID_FWD_MAX_SLOTS": 25, "BN_CL_GRID_BWD_MAX_SLOTS": 25},
       "bn_cl_grid_fwd_kernel", "bn_stats_cl_kernel"),
      ("above", ((256, 56, 56, 256), 3, F16), {"BN_CL_GRID_FWD_MAX_SLOTS": 120, "BN_CL_GRID_BWD_MAX_SLOTS": 120},
       "bn_stats_cl_kernel", "bn_cl_grid_fwd_kernel")]),
    # ... rows of 64-byte strips: backward up to 56 MiB in half, 16 MiB in float
    ("bn_cl_grid_narrow_bwd_max_kb", P.run_bn, {},
     [("below", ((320, 28, 28, 96), 3, F16), {"BN_CL_GRID_NARROW_BWD_MAX_KB": 1024}, "bn_cl_grid_bwd_kernel", "bn_bwd_reduce_cl_kernel"),
      ("above", ((560, 28, 28, 96), 3, F16), {"BN_CL_GRID_NARROW_BWD_MAX_KB": 1000000}, "bn_bwd_reduce_cl_kernel", "bn_cl_grid_bwd_kernel"),
      ("below_f32", ((48, 28, 28, 80), 3, F32), {"BN_CL_GRID_NARROW_BWD_MAX_KB_F32": 1024}, "bn_cl_grid_bwd_kernel", "bn_bwd_reduce_cl_kernel"),
      ("above_f32", ((200, 28, 28, 80), 3, F32), {"BN_CL_GRID_NARROW_BWD_MAX_KB_F32": 1000000}, "bn_bwd_reduce_cl_kernel", "bn_cl_grid_bwd_kernel")]),
    # short planes that share cache lines: ordinary stores inside the shared lines up to 1 KB
    ("bn_edge_stores_max_bytes", P.run_bn, NCS,
     [("below", ((256, 256, 14, 14), 1, F16), {"BN_EDGE_STORES_MAX_BYTES": 0}, "bn_onchip_fwd_kernel", "bn_onchip_fwd_kernel"),
      ("above", ((128, 256, 28, 28), 1, F16), {"BN_EDGE_STORES_MAX_BYTES": 4096}, "bn_onchip_fwd_kernel", "bn_onchip_fwd_kernel")]),
    # Group/InstanceNormalization rows that one block's registers hold as well
    # (up to 128 KB), held on one CU instead: from rows for 12 % of the CUs
    ("row_onchip_min_pct", P.run_in, {},
     [("below", (1, 24, (256, 256), F16), {"ROW_ONCHIP_MIN_PCT": 1}, "row_fwd_kernel", "row_onchip_fwd_kernel"),
      ("above", (1, 32, (256, 256), F16), {"ROW_ONCHIP_MIN_PCT": 100}, "row_onchip_fwd_kernel", "row_fwd_kernel")]),
    # ... longer rows (no register layout holds them): from the first row, both directions
    ("row_onchip_long_rows", P.run_in, {},
     [("few", (1, 8, (256, 256), F32), {"ROW_ONCHIP_MIN_PCT": 100, "ROW_ONCHIP_BWD_MIN_PCT": 100}, "row_onchip_fwd_kernel", "row_stats_stream_kernel"),
      ("more", (1, 56, (256, 256), F32), {"ROW_ONCHIP_MIN_PCT": 100, "ROW_ONCHIP_BWD_MIN_PCT": 100}, "bn_onchip_bwd_kernel", "plane_sums_stream_kernel")]),
    # ... rows beyond what a CU holds, the rest streamed: only with a row for nearly every CU
    ("row_onchip_streamed_min_pct", P.run_in, {},
     [("below", (1, 56, (512, 512), F32), {"ROW_ONCHIP_STREAMED_MIN_PCT": 1}, "row_stats_stream_kernel", "row_onchip_fwd_kernel")]),
    # rows held on one CU instead of in one block's registers: from 4097 vectors (beyond 64 KB;
    # the layouts of the on-chip kernel start at 5 vectors per thread, so only this side can be forced)
    ("row_onchip_fwd_min_vectors", P.run_gn, {},
     [("above", (16, 320, (64, 64), 32, F16), {"ROW_ONCHIP_FWD_MIN_VECTORS": 8193}, "row_onchip_fwd_kernel", "row_fwd_kernel")]),
    # GroupNormalization backward with the group on one CU: from 5 vectors per thread
    ("gn_onchip_bwd_min_nl", P.run_gn, {},
     [("below", (16, 256, (64, 64), 32, F16), {"GN_ONCHIP_BWD_MIN_NL": 4}, "row_bwd_kernel_gn", "gn_onchip_bwd_kernel"),
      ("above", (16, 320, (64, 64), 32, F16), {"GN_ONCHIP_BWD_MIN_NL": 9}, "gn_onchip_bwd_kernel", "row_bwd_kernel_gn")]),
    # channel-last groups that are no whole number of vectors: from 1 % of the CUs (3 blocks)
    ("gn_cl_tile_min_pct", P.run_gn, {},
     [("above", (4, 320, (8, 8), 32, F16, True), {"GN_CL_TILE_MIN_PCT": 100}, "gn_cl_tile_fwd_kernel", None)]),
    # channel-last groups of whole vectors off the 128-byte grid, beyond 4 MiB: the
    # position tiles ahead of the cached kernels from 2048 / 768 vectors per group
    ("gn_cl_tile_first", P.run_gn, {},
     [("below", (16, 200, (32, 32), 25, F16, True), {"GN_CL_TILE_FIRST_FWD": 0, "GN_CL_TILE_FIRST_BWD": 0},
       "gn_cl_row_fwd_kernel", "gn_cl_tile_fwd_kernel"),
      ("above", (16, 200, (48, 48), 25, F16, True), {"GN_CL_TILE_FIRST_FWD": 100000, "GN_CL_TILE_FIRST_BWD": 100000},
       "gn_cl_tile_fwd_kernel", "gn_cl_row_fwd_kernel"),
      ("below_f32", (64, 72, (16, 16), 9, F32, True), {"GN_CL_TILE_FIRST_FWD_F32": 0, "GN_CL_TILE_FIRST_BWD_F32": 0},
       "gn_cl_row_fwd_kernel", "gn_cl_tile_fwd_kernel"),
      ("above_f32", (32, 100, (40, 40), 25, F32, True),
       {"GN_CL_TILE_FIRST_FWD_F32": 100000, "GN_CL_TILE_FIRST_BWD_F32": 100000},
       "gn_cl_tile_fwd_kernel", "gn_cl_row_fwd_kernel")]),
    # channel-last InstanceNormalization beyond 4 MiB: cached instances up to 2048 positions
    ("in_cl_max", P.run_in, {},
     [("below", (40, 200, (40, 40), F16, True), {"IN_CL_MAX": 1024}, "in_cl_row_fwd_kernel", "bn_stats_cl_kernel"),
      ("above", (15, 200, (64, 64), F16, True), {"IN_CL_MAX": 8192}, "bn_stats_cl_kernel", "in_cl_row_fwd_kernel"),
      ("below_f32", (32, 100, (24, 24), F32, True), {"IN_CL_MAX_F32_FWD": 256, "IN_CL_MAX_F32_BWD": 256},
       "in_cl_row_fwd_kernel", "bn_stats_cl_kernel"),
      ("above_f32", (32, 100, (40, 40), F32, True), {"IN_CL_MAX_F32_FWD": 4096, "IN_CL_MAX_F32_BWD": 4096},
       "bn_stats_cl_kernel", "in_cl_row_fwd_kernel")]),
]
FLAT = [(cid, run, base, side) for cid, run, base, sides in CASES for side in sides]


@pytest.mark.parametrize("case", FLAT, ids=[f"{c[0]}-{c[3][0]}" for c in FLAT])
def test_threshold_crossover(case):
    cid, run, base, (side, args, forced, k_default, k_forced) = case
    timer = TIMERS[run]

    def under(knobs):
        names = P.kernels_of(run, args, knobs)           # parity against the oracle
        K.tune_reset()
        for name, value in knobs.items():
            K.tune_set(name, value)
        us, timed_names = timer(*args)
        K.tune_reset()
        return us, set(names) | set(timed_names)

    t_default, n_default = under(base)
    t_forced, n_forced = under({**base, **forced})
    if t_default > 1.15 * t_forced + 1.0:
        # (a measurement of a dozen calls can catch a hiccup of the box: one more
        # pair, the better time of each plan counts)
        t_default = min(t_default, under(base)[0])
        t_forced = min(t_forced, under({**base, **forced})[0])
    RESULTS[f"{cid}/{side}"] = {"shape": repr(args), "default_us": round(t_default, 2),
                                "other_plan_us": round(t_forced, 2), "forced_by": forced,
                                "default_kernels": sorted(n_default), "other_kernels": sorted(n_forced)}
    if k_default:
        assert k_default in n_default, (k_default, n_default)
    if k_forced:
        assert k_forced in n_forced, (k_forced, n_forced)
    if k_default != k_forced:
        assert n_default != n_forced, "the knob does not decide about this shape"
    assert t_default <= 1.15 * t_forced + 1.0, (
        f"{cid} {side} {args}: the default plan takes {t_default:.1f} us, the plan on the other "
        f"side of the threshold {t_forced:.1f} us")
