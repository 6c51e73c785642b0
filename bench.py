#!/usr/bin/env python3
"""Benchmark of the normalization hot path on one MI355X.

Headline workload (benchmark configuration 2): BatchNormalization training
forward + backward, fp32 NCHW x[32,256,56,56] ~ N(1,2), dy ~ N(0,1),
decay_rate 0.9, eps 1e-5.  One step = one forward (batch statistics, running
statistics update, y) plus one backward (dx, dgamma, dbeta) through the C-ABI,
inputs resident in HBM.

Cache honesty: MI355X has 256 MB of Infinity Cache behind 32 MB of L2, so a
loop over one set of buffers serves part of every call from cache - which a
training step, whose activations were written a whole network ago, never
sees.  Every workload here therefore owns several distinct sets of buffers
(real sizes, no flush kernel) and the timed loop walks them in turn, one lap
being four times L2 + Infinity Cache (1 GiB; --lap-mb); these "rotated" times are the ones
`value`, `roofline` and `pct_of_hbm_peak` are based on.  The same loop over
set 0 alone is reported beside them as `warm`.

Prints ONE JSON line.  `value` is algorithmic GB/s of the whole step (the
tensor passes the chosen plan makes: forward x + y with the channel held on
chip, else x twice + y; backward dy twice + dx + x once for the part of the
channel held on chip, twice for the rest); `roofline` is the kernel with the
most time per step, timed with HIP events on the launch stream in a second
region of the same K steps; `cpu_baseline` is the C restatement of the
reference arithmetic (oracle/norm_ref.c) on the same workload on the host
cores, all of them and one, priced with the same bytes as `value`, and it
also checks the outputs the timed GPU calls left behind against that
restatement; `configs` lists every benchmark configuration (microseconds per
call: mean of back-to-back calls, median and minimum over per-call event
pairs, and the warm mean).
"""
import argparse
import importlib.util
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# One lap over a workload's buffer sets must exceed L2 (8 x 4 MB) plus the
# Infinity Cache (256 MB) several times over: a cyclic walk of 1.2-1.4 times the
# cache still hits in it (measured: the 33 MB configurations and their plain
# copy run 10-35 % faster over a 352 MiB lap than over 1 GiB, and 2 GiB changes
# nothing further), so the default lap is 1 GiB.  --lap-mb sets another one.
# The buffer sets are counted so that the forward leg alone (x and y of every
# set in turn) walks a lap: sized by all four tensors of a set, the forward's
# own lap was 512 MiB and LayerNormalization [8192,4096] half ran it in 23 us
# against 33 us over 1 GiB.
LAP_BYTES = 1024 << 20


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def load_package():
    """Import nnabla-ext-cuda_amd/ (the directory name is not an identifier)."""
    name = "nnabla_ext_cuda_amd"
    if name in sys.modules:
        return sys.modules[name]
    pkg = os.path.join(ROOT, "nnabla-ext-cuda_amd")
    spec = importlib.util.spec_from_file_location(
        name, os.path.join(pkg, "__init__.py"), submodule_search_locations=[pkg])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


class Workload:
    """fwd(i) / bwd(i): one C-ABI call on buffer set i.  fwd_bytes/bwd_bytes:
    algorithmic bytes per call.  sets: the device buffers, one dict per set;
    host: the host copies of the inputs (for the parity check)."""

    def __init__(self, name, fwd, bwd, fwd_bytes, bwd_bytes, sets, host=None):
        self.name, self.fwd, self.bwd = name, fwd, bwd
        self.fwd_bytes, self.bwd_bytes = fwd_bytes, bwd_bytes
        self.sets, self.host = sets, host or {}

    @property
    def nsets(self):
        return len(self.sets)


def _ws(nbytes):
    import torch
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device="cuda")


def n_sets(bytes_per_set):
    return max(2, -(-LAP_BYTES // max(1, bytes_per_set)))


# Kernels that keep a BatchNormalization channel on chip (registers, LDS) and
# the tensor passes their direction then makes; the split reduction makes 3
# forward (x for the statistics, x again, y) and 5 backward.
BN_ONCHIP_FWD = ("bn_onchip_fwd_kernel", "row_fwd_kernel_bn", "in_cl_row_fwd_kernel",
                 "bn_cl_grid_fwd_kernel", "bn_pack_fwd_kernel", "bn_chan_split_fwd_kernel")
BN_ONCHIP_BWD = {"bn_onchip_bwd_kernel": 4, "row_bwd_kernel_bn": 3, "in_cl_row_bwd_kernel": 3,
                 "bn_pack_bwd_kernel": 3, "bn_chan_split_bwd_kernel": 3}
# bn_onchip_bwd_kernel holds x of a channel on its CU and streams dy twice
# (x, 2 dy, dx = 4 passes); of a channel beyond 20480 16-byte vectors it holds
# 18432 from the start plus 3072 parked in LDS on their way through the first
# pass, and reads the rest of x twice as well.
BN_ONCHIP_BWD_HELD, BN_ONCHIP_BWD_WHOLE = 18432 + 3072, 20480
# bn_onchip_fwd_kernel holds up to 25600 vectors of a channel; the rest of a
# longer channel is read twice.
BN_ONCHIP_FWD_HELD = 25600


# bn_cl_grid_bwd_kernel (channel-last, the whole tensor on the chip's 256 CUs)
# holds 21 x 1024 vectors of x per block and reads what a block has beyond that
# twice, like dy: x, 2 dy, dx = 4 passes + the part of x not held.
BN_CL_GRID_BWD_HELD, BN_CL_GRID_BLOCKS = 21 * 1024, 256


def bn_tensor_passes(K, fwd, bwd, vectors_per_channel=0, channel_last_vectors=0):
    """(forward, backward) tensor passes of the plan the library picks for this
    workload: a pass counts when the channel cannot stay on chip between the
    statistics and the apply phase.  Read off the kernels one call launches."""
    import torch
    L = K.lib()
    K.check(L.nblahip_profile_enable(64))
    fwd(0)
    bwd(0)
    torch.cuda.synchronize()
    pf = 2 if any(K.profile_query(k)[1] for k in BN_ONCHIP_FWD) else 3
    if K.profile_query("bn_onchip_fwd_kernel")[1] and vectors_per_channel > BN_ONCHIP_FWD_HELD:
        pf += (vectors_per_channel - BN_ONCHIP_FWD_HELD) / vectors_per_channel
    pb = 5
    for k, passes in BN_ONCHIP_BWD.items():
        if K.profile_query(k)[1]:
            pb = passes
            if k == "bn_onchip_bwd_kernel" and vectors_per_channel > BN_ONCHIP_BWD_WHOLE:
                pb += (vectors_per_channel - BN_ONCHIP_BWD_HELD) / vectors_per_channel
    if K.profile_query("bn_cl_grid_bwd_kernel")[1]:
        per_block = -(-channel_last_vectors // BN_CL_GRID_BLOCKS)
        pb = 4 + max(0, per_block - BN_CL_GRID_BWD_HELD) / max(1, per_block)
    K.check(L.nblahip_profile_enable(0))
    return pf, pb


def _np_dtype(dtype):
    import torch
    return np.float16 if dtype == torch.float16 else np.float32


def make_bn(K, name, shape, axis, dtype, train, mean=0.0, std=1.0, outliers=False, seed=0,
            fused=False, stream=None, rotate=True):
    """BatchNormalization workload.  Inputs are drawn on the host from
    numpy.random.default_rng(seed) in the order the full-size parity tests
    draw them (x, [outlier mask], dy, gamma, beta), so both see the same data."""
    import torch
    L = K.lib()
    rng = np.random.default_rng(seed)
    c = shape[axis]
    npdt = _np_dtype(dtype)
    if train:
        x = rng.standard_normal(shape, dtype=np.float32)
        if std != 1.0 or mean != 0.0:
            x = (x * std + mean).astype(np.float32)
        if outliers:
            mask = rng.random(shape, dtype=np.float32) < 0.01
            x = np.where(mask, x * 50, x)
            del mask
        x = x.astype(npdt)
        dy = rng.standard_normal(shape, dtype=np.float32).astype(npdt)
        gamma = rng.uniform(0.5, 1.5, c).astype(np.float32)
        beta = (rng.standard_normal(c) * 0.1).astype(np.float32)
        rm0, rv0 = np.zeros(c, np.float32), np.ones(c, np.float32)
        z = rng.standard_normal(shape, dtype=np.float32).astype(npdt) if fused else None
    else:
        x = rng.standard_normal(shape).astype(np.float32).astype(npdt)
        dy = z = None
        gamma = rng.uniform(0.5, 1.5, c).astype(np.float32)
        beta = (rng.standard_normal(c) * 0.1).astype(np.float32)
        rm0 = (rng.standard_normal(c) * 0.1).astype(np.float32)
        rv0 = rng.uniform(0.5, 2, c).astype(np.float32)
    host = {"x": x, "dy": dy, "gamma": gamma, "beta": beta, "rm": rm0, "rv": rv0}
    S = x.nbytes
    # (sized by what the forward alone touches - x, y and the fused z: every leg
    # timed on its own must walk a whole lap too)
    per_set = S * ((3 if fused else 2) if train else 2)
    sets = []
    up = lambda a: None if a is None else torch.from_numpy(a).cuda()
    gd, bd = up(gamma), up(beta)
    for i in range(n_sets(per_set) if rotate else 1):
        first = sets[0] if sets else None
        s = {"x": up(x) if first is None else first["x"].clone(),
             "dy": (up(dy) if first is None else first["dy"].clone()) if train else None,
             "z": (up(z) if first is None else first["z"].clone()) if fused else None,
             "rm": up(rm0), "rv": up(rv0)}
        s["y"] = torch.empty_like(s["x"])
        if train:
            s["dx"] = torch.empty_like(s["x"])
            s["dz"] = torch.empty_like(s["x"]) if fused else None
            for k in ("bm", "bv", "dg", "db"):
                s[k] = torch.empty(c, device="cuda")
        sets.append(s)
    s0, _, s2 = K._bn_sizes(shape, axis)
    dt = K._dtype_code(sets[0]["x"])
    ws = _ws(L.nblahip_bn_workspace_bytes(s0, c, s2, dt))
    st = stream if stream is not None else torch.cuda.current_stream().cuda_stream
    n = len(sets)
    P = [{k: (None if v is None else v.data_ptr()) for k, v in s.items()} for s in sets]
    g_p, b_p, ws_p, ws_n = gd.data_ptr(), bd.data_ptr(), ws.data_ptr(), ws.numel()
    keep = (sets, gd, bd, ws)

    if train and fused:
        # FusedBatchNormalization: y = relu(bn(x) + z); backward also yields dz.
        def fwd(i):
            p = P[i % n]
            K.check(L.nblahip_fused_bn_fwd_train(p["x"], p["z"], g_p, b_p, p["y"], p["bm"], p["bv"],
                                                 p["rm"], p["rv"], s0, c, s2, 0.9, 1e-5, dt, ws_p,
                                                 ws_n, st))

        def bwd(i):
            p = P[i % n]
            K.check(L.nblahip_fused_bn_bwd(p["x"], p["y"], p["dy"], g_p, p["bm"], p["bv"], None,
                                           None, p["dx"], p["dz"], p["dg"], p["db"], 0, 0, 0, 0, s0,
                                           c, s2, 1e-5, 1, dt, ws_p, ws_n, st))
        # fwd: x (stats), x, z (apply), y; bwd: x, dy, y, dz (reduce), x, dz, dx (apply)
        w = Workload(name, fwd, bwd, 4 * S, 7 * S, sets, host)
    elif train:
        def fwd(i):
            p = P[i % n]
            K.check(L.nblahip_bn_fwd_train(p["x"], g_p, b_p, p["y"], p["bm"], p["bv"], p["rm"],
                                           p["rv"], s0, c, s2, 0.9, 1e-5, dt, ws_p, ws_n, st))

        def bwd(i):
            p = P[i % n]
            K.check(L.nblahip_bn_bwd(p["x"], p["dy"], g_p, p["bm"], p["bv"], None, None, p["dx"],
                                     p["dg"], p["db"], 0, 0, 0, s0, c, s2, 1e-5, 1, dt, ws_p, ws_n,
                                     st))
        # (vectors are 16 bytes, 8 for half planes of 4k - not 8k - elements)
        esz = sets[0]["x"].element_size()
        vec_bytes = 8 if esz == 2 and s2 % 8 != 0 and s2 % 4 == 0 else 16
        pf, pb = bn_tensor_passes(K, fwd, bwd, s0 * s2 * esz // vec_bytes,
                                  s0 * c * esz // 16 if s2 == 1 else 0)
        # the probe call moved the running statistics of set 0: start over
        sets[0]["rm"].copy_(up(rm0))
        sets[0]["rv"].copy_(up(rv0))
        w = Workload(name, fwd, bwd, int(round(pf * S)), int(round(pb * S)), sets, host)
        w.passes = (pf, pb)
    else:
        def fwd(i):
            p = P[i % n]
            K.check(L.nblahip_bn_fwd_infer(p["x"], p["rm"], p["rv"], g_p, b_p, p["y"], s0, c, s2,
                                           1e-5, dt, st))
        w = Workload(name, fwd, None, 2 * S, 0, sets, host)
    w.keep = keep
    return w


def make_rows(K, name, kind, shape, dtype, seed, rotate=True, **kw):
    """kind in {"ln", "gn", "in"}; shape [outer..., R] for ln, [N,C,H,W] else
    ([N,H,W,C] with channel_last=True).  Host-drawn inputs as in make_bn."""
    import torch
    L = K.lib()
    rng = np.random.default_rng(seed)
    npdt = _np_dtype(dtype)
    x = rng.standard_normal(shape, dtype=np.float32) * np.float32(kw.get("std", 1.0))
    if kind == "ln":
        x = x + rng.uniform(-3, 3, shape[:-1] + (1,)).astype(np.float32)
    x = x.astype(npdt)
    dy = rng.standard_normal(shape, dtype=np.float32).astype(npdt)
    S = x.nbytes
    up = lambda a: torch.from_numpy(a).cuda()
    cl = kw.get("channel_last", False)
    if kind == "ln":
        R = shape[-1]
        outer = x.size // R
        gamma = (rng.standard_normal(R) * 0.1 + 1).astype(np.float32)
        beta = (rng.standard_normal(R) * 0.1).astype(np.float32)
        nstat, nparam = outer, R
    else:
        nb, c = shape[0], shape[-1] if cl else shape[1]
        sp = x.size // (nb * c)
        gamma = rng.uniform(0.5, 1.5, c).astype(np.float32)
        beta = (rng.standard_normal(c) * 0.1).astype(np.float32)
        nstat, nparam = (nb * kw["groups"] if kind == "gn" else nb * c), c
    gd, bd = up(gamma), up(beta)
    sets = []
    for i in range(n_sets(2 * S) if rotate else 1):  # (x and y: what the forward leg touches)
        first = sets[0] if sets else None
        s = {"x": up(x) if first is None else first["x"].clone(),
             "dy": up(dy) if first is None else first["dy"].clone()}
        s["y"], s["dx"] = torch.empty_like(s["x"]), torch.empty_like(s["x"])
        s["mean"], s["var"] = torch.empty(nstat, device="cuda"), torch.empty(nstat, device="cuda")
        s["dg"], s["db"] = torch.empty(nparam, device="cuda"), torch.empty(nparam, device="cuda")
        sets.append(s)
    dt = K._dtype_code(sets[0]["x"])
    st = torch.cuda.current_stream().cuda_stream
    n = len(sets)
    P = [{k: v.data_ptr() for k, v in s.items()} for s in sets]
    g_p, b_p = gd.data_ptr(), bd.data_ptr()
    if kind == "ln":
        ws = _ws(L.nblahip_ln_bwd_workspace_bytes(outer, R, dt))
        ws_p, ws_n = ws.data_ptr(), ws.numel()

        def fwd(i):
            p = P[i % n]
            K.check(L.nblahip_ln_fwd(p["x"], g_p, b_p, p["y"], p["mean"], p["var"], outer, R, 1e-5,
                                     dt, st))

        def bwd(i):
            p = P[i % n]
            K.check(L.nblahip_ln_bwd(p["x"], p["dy"], g_p, p["mean"], p["var"], None, None, p["dx"],
                                     p["dg"], p["db"], 0, 0, 0, outer, R, 1e-5, dt, ws_p, ws_n, st))
    elif kind == "gn":
        G = kw["groups"]
        ws = _ws(L.nblahip_gn_cl_workspace_bytes(nb, sp, c, G, dt) if cl else
                 L.nblahip_gn_bwd_workspace_bytes(nb, c, sp, G, dt))
        ws_p, ws_n = ws.data_ptr(), ws.numel()
        if cl:
            def fwd(i):
                p = P[i % n]
                K.check(L.nblahip_gn_cl_fwd(p["x"], g_p, b_p, p["y"], p["mean"], p["var"], nb, sp, c,
                                            G, 1e-5, dt, ws_p, ws_n, st))

            def bwd(i):
                p = P[i % n]
                K.check(L.nblahip_gn_cl_bwd(p["x"], p["dy"], g_p, p["mean"], p["var"], None, None,
                                            p["dx"], p["dg"], p["db"], 0, 0, 0, nb, sp, c, G, 1e-5,
                                            dt, ws_p, ws_n, st))
        else:
            def fwd(i):
                p = P[i % n]
                K.check(L.nblahip_gn_fwd(p["x"], g_p, b_p, p["y"], p["mean"], p["var"], nb, c, sp, G,
                                         1e-5, dt, st))

            def bwd(i):
                p = P[i % n]
                K.check(L.nblahip_gn_bwd(p["x"], p["dy"], g_p, p["mean"], p["var"], None, None,
                                         p["dx"], p["dg"], p["db"], 0, 0, 0, nb, c, sp, G, 1e-5, dt,
                                         ws_p, ws_n, st))
    else:
        ws = _ws(L.nblahip_in_cl_workspace_bytes(nb, sp, c, dt) if cl else
                 L.nblahip_in_bwd_workspace_bytes(nb, c, sp, dt))
        ws_p, ws_n = ws.data_ptr(), ws.numel()
        if cl:
            def fwd(i):
                p = P[i % n]
                K.check(L.nblahip_in_cl_fwd(p["x"], g_p, b_p, p["y"], p["mean"], p["var"], nb, sp, c,
                                            1, 1, 1e-5, dt, ws_p, ws_n, st))

            def bwd(i):
                p = P[i % n]
                K.check(L.nblahip_in_cl_bwd(p["x"], p["dy"], g_p, p["mean"], p["var"], None, None,
                                            p["dx"], p["dg"], p["db"], 0, 0, 0, nb, sp, c, 1, 1,
                                            1e-5, dt, ws_p, ws_n, st))
        else:
            def fwd(i):
                p = P[i % n]
                K.check(L.nblahip_in_fwd(p["x"], g_p, b_p, p["y"], p["mean"], p["var"], nb, c, sp, 1,
                                         1, 1e-5, dt, st))

            def bwd(i):
                p = P[i % n]
                K.check(L.nblahip_in_bwd(p["x"], p["dy"], g_p, p["mean"], p["var"], None, None,
                                         p["dx"], p["dg"], p["db"], 0, 0, 0, nb, c, sp, 1, 1, 1e-5,
                                         dt, ws_p, ws_n, st))
    w = Workload(name, fwd, bwd, 2 * S, 3 * S, sets, {"x": x, "dy": dy, "gamma": gamma, "beta": beta})
    w.keep = (sets, gd, bd, ws)
    return w


def time_calls(fns, steps, warmup, rotate=True):
    """Wall-clock milliseconds per step of calling every fn in fns once, back to
    back; step k works on buffer set k (rotate) or on set 0."""
    import torch
    for k in range(warmup):
        for f in fns:
            f(k if rotate else 0)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(steps):
        for f in fns:
            f(k if rotate else 0)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def time_events(fns, steps):
    """(median, min) microseconds per step from one HIP event pair around every
    step (recorded on the stream the calls launch on), buffer sets in turn."""
    import torch
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
          for _ in range(steps)]
    for k in range(steps):
        ev[k][0].record()
        for f in fns:
            f(k)
        ev[k][1].record()
    torch.cuda.synchronize()
    us = [a.elapsed_time(b) * 1e3 for a, b in ev]
    return statistics.median(us), min(us)


def time_in_graph(K, calls, steps, warmup):
    """Milliseconds per call of the C1 inference forward when `calls` of them
    are captured into one graph and the graph is replayed."""
    import torch
    side = torch.cuda.Stream()
    w = make_bn(K, "C1", (8, 64, 56, 56), 1, torch.float32, False, seed=0,
                stream=side.cuda_stream, rotate=False)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        w.fwd(0)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for _ in range(calls):
                w.fwd(0)
    ms = time_calls([lambda i: graph.replay()], max(1, steps // 4), max(1, warmup // 4)) / calls
    del graph, w
    return ms


def config_specs(K):
    import torch
    f32, f16 = torch.float32, torch.float16
    return [
        ("C1 BN inference fp32 [8,64,56,56]", lambda n: make_bn(K, n, (8, 64, 56, 56), 1, f32, False, seed=0)),
        ("C2 BN training fp32 NCHW [32,256,56,56]", lambda n: make_bn(K, n, (32, 256, 56, 56), 1, f32, True, 1.0, 2.0, seed=1)),
        ("C3 LN fp32 [32,512,1024]", lambda n: make_rows(K, n, "ln", (32, 512, 1024), f32, 2)),
        ("C3 LN fp16 [32,512,1024]", lambda n: make_rows(K, n, "ln", (32, 512, 1024), f16, 2)),
        ("C4 GN fp16 [16,256,64,64] G=32", lambda n: make_rows(K, n, "gn", (16, 256, 64, 64), f16, 3, std=1.5, groups=32)),
        ("C4 IN fp16 [16,256,64,64]", lambda n: make_rows(K, n, "in", (16, 256, 64, 64), f16, 3, std=1.5)),
        ("C4 GN fp16 NHWC [16,64,64,256] G=32", lambda n: make_rows(K, n, "gn", (16, 64, 64, 256), f16, 3, std=1.5, groups=32, channel_last=True)),
        ("C4 IN fp16 NHWC [16,64,64,256]", lambda n: make_rows(K, n, "in", (16, 64, 64, 256), f16, 3, std=1.5, channel_last=True)),
        ("C5 BN training fp16 NHWC [256,56,56,64]", lambda n: make_bn(K, n, (256, 56, 56, 64), 3, f16, True, outliers=True, seed=4)),
        ("Fused BN+add+ReLU training fp16 NHWC [256,56,56,64]", lambda n: make_bn(K, n, (256, 56, 56, 64), 3, f16, True, outliers=True, seed=4, fused=True)),
    ]


def config_table(K, steps, warmup, only=None):
    """Every benchmark configuration: microseconds per call (rotated buffer
    sets: mean of back-to-back calls, median and minimum of per-call event
    pairs; warm: mean over one buffer set) and algorithmic GB/s of the rotated
    mean."""
    import torch
    out = []
    for name, make in config_specs(K):
        if only and only not in name:
            continue
        w = make(name)
        row = {"config": name, "buffer_sets": w.nsets,
               "lap_bytes": sum(t.numel() * t.element_size() for s_ in w.sets
                                for t in s_.values() if t is not None)}
        legs = [("fwd", [w.fwd], w.fwd_bytes)]
        if w.bwd is not None:
            legs += [("bwd", [w.bwd], w.bwd_bytes), ("fwd_bwd", [w.fwd, w.bwd], w.fwd_bytes + w.bwd_bytes)]
        for key, fns, nbytes in legs:
            ms = time_calls(fns, steps, warmup)
            med, mn = time_events(fns, steps)
            warm = time_calls(fns, steps, warmup, rotate=False)
            row[key + "_us"] = round(ms * 1e3, 2)
            row[key + "_median_us"] = round(med, 2)
            row[key + "_min_us"] = round(mn, 2)
            row[key + "_warm_us"] = round(warm * 1e3, 2)
            row[key + "_GBps"] = round(nbytes / ms / 1e6, 1)
        last = legs[-1][0]
        # What the memory system gives a plain copy of one tensor of this size
        # in the same rotated loop (x -> y of every buffer set in turn, 2 S per
        # call): the practical ceiling beside the 8 TB/s of the data sheet.
        def plain_copy(i, sets=w.sets):
            b = sets[i % len(sets)]
            b["y"].copy_(b["x"], non_blocking=True)
        x0 = w.sets[0]["x"]
        cms = time_calls([plain_copy], steps, warmup)
        row["copy_us"] = round(cms * 1e3, 2)
        row["copy_GBps"] = round(2 * x0.numel() * x0.element_size() / cms / 1e6, 1)
        row["pct_of_copy_speed"] = round(row[last + "_GBps"] / row["copy_GBps"] * 100, 1)
        if w.bwd is not None:
            row["pct_of_hbm_peak"] = round(row[last + "_GBps"] / HBM_PEAK_GBS * 100, 1)
            row["pct_of_hbm_peak_warm"] = round(
                legs[-1][2] / row[last + "_warm_us"] / 1e3 / HBM_PEAK_GBS * 100, 1)
        else:
            # A 13 MB pass is bounded by the cost of a dispatch, not by bytes:
            # the same call replayed from a captured graph of 20 calls, per call.
            row["bound"] = "launch"
            row["fwd_us_in_graph"] = round(time_in_graph(K, 20, steps, warmup) * 1e3, 2)
        log("  ", json.dumps(row))
        out.append(row)
        del w
        torch.cuda.empty_cache()
    return out


def torch_native_table(K, steps, warmup):
    """This library beside the framework's own kernels on the same GPU:
    torch.ops.aten.native_{batch,layer,group}_norm and their backward ops on the
    same shapes (wall clock per call, microseconds, one buffer set each)."""
    import torch
    A = torch.ops.aten

    def bn(shape, dt, cl):
        n, c, h, w = shape
        x = torch.randn(shape, device="cuda", dtype=dt)
        dy = torch.randn_like(x)
        if cl:
            x = x.contiguous(memory_format=torch.channels_last)
            dy = dy.contiguous(memory_format=torch.channels_last)
        g, b = torch.rand(c, device="cuda") + 0.5, torch.randn(c, device="cuda")
        rm, rv = torch.zeros(c, device="cuda"), torch.ones(c, device="cuda")
        fwd_t = lambda: A.native_batch_norm(x, g, b, rm, rv, True, 0.1, 1e-5)
        _, sm, si = fwd_t()
        bwd_t = lambda: A.native_batch_norm_backward(dy, x, g, rm, rv, sm, si, True, 1e-5,
                                                     [True, True, True])
        ours = make_bn(K, "", (n, h, w, c) if cl else shape, 3 if cl else 1, dt, True, seed=1,
                       rotate=False)
        return fwd_t, bwd_t, ours

    def ln(shape, dt):
        rows, r = shape
        x = torch.randn(shape, device="cuda", dtype=dt)
        dy = torch.randn_like(x)
        g, b = (torch.rand(r, device="cuda") + 0.5).to(dt), torch.randn(r, device="cuda").to(dt)
        fwd_t = lambda: A.native_layer_norm(x, [r], g, b, 1e-5)
        _, m, rs = fwd_t()
        bwd_t = lambda: A.native_layer_norm_backward(dy, x, [r], m, rs, g, b, [True, True, True])
        return fwd_t, bwd_t, make_rows(K, "", "ln", shape, dt, 3, rotate=False)

    def gn(shape, groups, dt):
        n, c, h, w = shape
        x = torch.randn(shape, device="cuda", dtype=dt)
        dy = torch.randn_like(x)
        g, b = (torch.rand(c, device="cuda") + 0.5).to(dt), torch.randn(c, device="cuda").to(dt)
        fwd_t = lambda: A.native_group_norm(x, g, b, n, c, h * w, groups, 1e-5)
        _, m, rs = fwd_t()
        bwd_t = lambda: A.native_group_norm_backward(dy, x, m, rs, g, n, c, h * w, groups,
                                                     [True, True, True])
        ours = (make_rows(K, "", "in", shape, dt, 3, rotate=False) if groups == c
                else make_rows(K, "", "gn", shape, dt, 3, groups=groups, rotate=False))
        return fwd_t, bwd_t, ours

    f32, f16 = torch.float32, torch.float16
    specs = []
    for dt in (f32, f16):
        n = str(dt)[6:]
        specs += [
            (f"BN {n} NCHW [32,256,56,56]", lambda dt=dt: bn((32, 256, 56, 56), dt, False)),
            (f"BN {n} NHWC [256,56,56,64]", lambda dt=dt: bn((256, 64, 56, 56), dt, True)),
            (f"BN {n} NCHW [256,1024,14,14]", lambda dt=dt: bn((256, 1024, 14, 14), dt, False)),
            (f"BN {n} NCHW [256,2048,7,7]", lambda dt=dt: bn((256, 2048, 7, 7), dt, False)),
            (f"LN {n} [16384,1024]", lambda dt=dt: ln((16384, 1024), dt)),
            (f"LN {n} [8192,4096]", lambda dt=dt: ln((8192, 4096), dt)),
            (f"LN {n} [262144,128]", lambda dt=dt: ln((262144, 128), dt)),
            (f"GN {n} [16,256,64,64] G=32", lambda dt=dt: gn((16, 256, 64, 64), 32, dt)),
            (f"GN {n} [32,512,28,28] G=32", lambda dt=dt: gn((32, 512, 28, 28), 32, dt)),
            (f"GN {n} [32,1024,14,14] G=32", lambda dt=dt: gn((32, 1024, 14, 14), 32, dt)),
            (f"IN {n} [16,256,64,64]", lambda dt=dt: gn((16, 256, 64, 64), 256, dt)),
        ]
    out = []
    for name, make in specs:
        fwd_t, bwd_t, w = make()
        row = {"config": name}
        for key, ours, theirs in (("fwd", w.fwd, fwd_t), ("bwd", w.bwd, bwd_t)):
            a = time_calls([ours], steps, warmup, rotate=False) * 1e3
            b = time_calls([lambda i: theirs()], steps, warmup, rotate=False) * 1e3
            row[key + "_us"] = round(a, 1)
            row["torch_" + key + "_us"] = round(b, 1)
            row[key + "_speedup"] = round(b / a, 2)
        log("  ", json.dumps(row))
        out.append(row)
        del w, fwd_t, bwd_t
        torch.cuda.empty_cache()
    return out


def _worst(got, ref, rtol, atol):
    """max |got-ref| / (atol + rtol*|ref|): <= 1 means within tolerance."""
    got = np.asarray(got, np.float64).reshape(-1)
    ref = np.asarray(ref, np.float64).reshape(-1)
    return float(np.max(np.abs(got - ref) / (atol + rtol * np.abs(ref))))


def cpu_baseline(host, gpu_out, step_bytes, budget_s=12.0):
    """The C restatement of the reference arithmetic on the full C2 workload:
    timed with OpenMP over all host threads and with one thread, and used as
    the checker of what the timed GPU calls left in their output buffers
    (fp32: rel 1e-5 / abs 1e-5; dgamma/dbeta with the absolute floor scaled by
    max(1, RMS) of the vector, as in the parity tests)."""
    from oracle import c_ref as C
    x, dy, g, b = host["x"], host["dy"], host["gamma"], host["beta"]
    n0, c, hw = x.shape[0], x.shape[1], x.shape[2] * x.shape[3]
    lib = C.lib()
    cores = lib.nr_num_threads()

    def step():
        rm, rv = np.zeros(c, np.float32), np.ones(c, np.float32)
        y, m, v = C.bn_forward_batch(x, b, g, rm, rv, n0, c, hw, 0.9, 1e-5)
        dx, dg, db = C.bn_backward_batch(x, dy, g, m, v, n0, c, hw, 1e-5)
        return {"y": y, "mean": m, "var": v, "dx": dx, "dgamma": dg, "dbeta": db}

    def timed(max_reps, budget):
        reps, total, out = 0, 0.0, None
        while reps < max_reps and (reps == 0 or total < budget):
            t0 = time.perf_counter()
            out = step()
            total += time.perf_counter() - t0
            reps += 1
        return total / reps, reps, out

    sec, reps, ref = timed(20, budget_s)
    lib.nr_set_num_threads(1)
    sec1, reps1, _ = timed(3, 6.0)
    lib.nr_set_num_threads(cores)

    parity = None
    if gpu_out is not None:
        parity = {}
        for k in ("y", "mean", "var", "dx"):
            parity[k] = round(_worst(gpu_out[k], ref[k], 1e-5, 1e-5), 3)
        for k in ("dgamma", "dbeta"):
            rms = float(np.sqrt(np.mean(np.asarray(ref[k], np.float64) ** 2)))
            parity[k] = round(_worst(gpu_out[k], ref[k], 1e-5, 1e-5 * max(1.0, rms)), 3)
        parity["ok"] = bool(all(v <= 1.0 for v in parity.values()))
        parity["note"] = ("worst |gpu - cpu| / (atol + rtol*|cpu|) per output of the timed GPU "
                          "calls (buffer set 0) against this restatement; <= 1 is within tolerance")
    return {"value": round(step_bytes / sec / 1e9, 3), "unit": "GB/s", "cores": int(cores),
            "kind": "port", "ms_per_step": round(sec * 1e3, 2),
            "single_thread": {"value": round(step_bytes / sec1 / 1e9, 3), "unit": "GB/s",
                              "cores": 1, "ms_per_step": round(sec1 * 1e3, 2), "repetitions": reps1},
            "bytes_per_step": step_bytes,
            "sample": f"full workload x[32,256,56,56] fwd+bwd, {reps} repetitions, "
                      f"oracle/norm_ref.c with OpenMP over channels; GB/s priced with the GPU "
                      f"step's algorithmic bytes",
            "parity": parity}


TRAFFIC_FILE = os.path.join("profiles", "c2_kernel_traffic.txt")


def load_traffic(kernel):
    """HBM bytes per launch of a kernel of the headline workload from the
    committed rocprofv3 --pmc summary (FETCH_SIZE and WRITE_SIZE scaled by a
    convert kernel of known traffic), or None."""
    try:
        with open(os.path.join(ROOT, TRAFFIC_FILE)) as f:
            return json.load(f).get(kernel, {}).get("hbm_bytes_per_launch")
    except (OSError, ValueError):
        return None


def main():
    global LAP_BYTES
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-table", action="store_true", help="skip the per-config table")
    ap.add_argument("--only", default=None, help="table rows whose name contains this text")
    ap.add_argument("--table-only", action="store_true",
                    help="only the per-configuration table (with --only: a few rows), printed as "
                         "one JSON line {\"configs\": [...]}; no headline workload, no CPU "
                         "baseline - the short command for per-kernel counter runs")
    ap.add_argument("--torch-native", action="store_true",
                    help="also time torch's own normalization kernels on the same shapes")
    ap.add_argument("--lap-mb", type=int, default=LAP_BYTES >> 20,
                    help="bytes (MiB) one lap over a workload's rotated buffer sets must exceed")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch a float32->float16 convert of the workload's x (a plain "
                         "streaming kernel of known traffic: 4 B read, 2 B written per element) "
                         "so that rocprofv3 --pmc FETCH_SIZE/WRITE_SIZE readings can be scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus must be 1 (the path shards by "
              "batch; the exchange between shards belongs to the caller's communicator)",
              file=sys.stderr)
        sys.exit(2)

    LAP_BYTES = max(1, args.lap_mb) << 20

    import torch
    K = load_package()
    L = K.lib()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)

    if args.table_only:
        print(json.dumps({"lap_floor_bytes": LAP_BYTES, "steps": args.steps,
                          "configs": config_table(K, args.steps, args.warmup, args.only)}),
              flush=True)
        return

    name = ("BatchNormalization training fwd+bwd fp32 NCHW x[32,256,56,56] "
            "(benchmark configuration 2), decay_rate 0.9, eps 1e-5")
    w = make_bn(K, name, (32, 256, 56, 56), 1, torch.float32, True, 1.0, 2.0, seed=1)
    fb, bb = w.fwd_bytes, w.bwd_bytes
    if args.calibrate:
        xs = w.sets[0]["x"]
        half = torch.empty(xs.shape, dtype=torch.float16, device="cuda")
        st = torch.cuda.current_stream().cuda_stream
        for _ in range(args.steps):
            K.check(L.nblahip_convert(half.data_ptr(), K.F16, xs.data_ptr(), K.F32, xs.numel(), st))
        torch.cuda.synchronize()
        del half
    ms = time_calls([w.fwd, w.bwd], args.steps, args.warmup)
    med_us, min_us = time_events([w.fwd, w.bwd], args.steps)
    warm_ms = time_calls([w.fwd, w.bwd], args.steps, args.warmup, rotate=False)
    value = (fb + bb) / ms / 1e6  # GB/s
    log(f"C2 fwd+bwd: {ms * 1e3:.1f} us/step over {w.nsets} buffer sets ({value:.0f} GB/s "
        f"algorithmic; median {med_us:.1f}, min {min_us:.1f}), {warm_ms * 1e3:.1f} us on one set")

    # Second region: the same K steps with per-kernel HIP events.
    kernels = ["bn_onchip_fwd_kernel", "bn_onchip_bwd_kernel",
               "bn_stats_planes_kernel", "bn_finalize_fwd_kernel", "bn_apply_planes_kernel",
               "bn_apply_planes_fused_kernel", "bn_bwd_reduce_planes_kernel",
               "bn_finalize_bwd_kernel", "bn_bwd_apply_planes_kernel",
               "bn_bwd_apply_planes_fused_kernel"]
    K.check(L.nblahip_profile_enable(args.steps * len(kernels) + 16))
    for k in range(args.steps):
        w.fwd(k)
        w.bwd(k)
    torch.cuda.synchronize()
    S = w.host["x"].nbytes
    kbytes = {"bn_onchip_fwd_kernel": fb, "bn_onchip_bwd_kernel": bb,
              "bn_stats_planes_kernel": S, "bn_apply_planes_kernel": 2 * S,
              "bn_apply_planes_fused_kernel": 2 * S, "bn_bwd_reduce_planes_kernel": 2 * S,
              "bn_bwd_apply_planes_kernel": 3 * S, "bn_bwd_apply_planes_fused_kernel": 3 * S}
    per_kernel = {}
    for k in kernels:
        tot, cnt = K.profile_query(k)
        if cnt:
            per_kernel[k] = {"avg_us": round(tot / cnt * 1e3, 2), "launches": cnt}
            if k in kbytes:
                per_kernel[k]["GBps"] = round(kbytes[k] / (tot / cnt) / 1e6, 1)
    K.check(L.nblahip_profile_enable(0))
    log("per-kernel:", json.dumps(per_kernel))
    # dominant kernel = the one with the most time per step
    dom = max((k for k in per_kernel if k in kbytes), key=lambda k: per_kernel[k]["avg_us"])
    achieved = per_kernel[dom]["GBps"]
    roofline = {"bound": "hbm", "kernel": dom, "achieved": achieved, "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                "avg_us": per_kernel[dom]["avg_us"], "algorithmic_bytes": kbytes[dom],
                "traffic": load_traffic(dom),
                "traffic_source": TRAFFIC_FILE + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of "
                                                 "this command, read from the committed summary, "
                                                 "not measured in this run)"}

    pf, pb = w.passes
    result = {
        "metric": "BN training fwd+bwd achieved algorithmic HBM bandwidth (us/call in ms_per_step), 1 MI355X",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": name,
                   "algorithmic_bytes_per_step": fb + bb,
                   "tensor_passes": {"forward": round(pf, 3), "backward": round(pb, 3),
                                     "note": "a pass counts when the channel cannot stay on chip "
                                             "between statistics and apply"},
                   "buffer_sets": w.nsets,
                   "lap_bytes": w.nsets * 4 * S,
                   "lap_floor_bytes": LAP_BYTES,
                   "median_us": round(med_us, 2), "min_us": round(min_us, 2),
                   "warm_ms_per_step": round(warm_ms, 5),
                   "warm_GBps": round((fb + bb) / warm_ms / 1e6, 1),
                   "pct_of_hbm_peak": round(value / HBM_PEAK_GBS * 100, 1)},
        "roofline": roofline,
        "per_kernel": per_kernel,
    }
    gpu_out = None
    if not args.no_cpu:
        # what the timed calls left in buffer set 0
        s = w.sets[0]
        gpu_out = {"y": s["y"].cpu().numpy(), "mean": s["bm"].cpu().numpy(),
                   "var": s["bv"].cpu().numpy(), "dx": s["dx"].cpu().numpy(),
                   "dgamma": s["dg"].cpu().numpy(), "dbeta": s["db"].cpu().numpy()}
    host = w.host
    del w
    torch.cuda.empty_cache()
    if not args.no_table:
        result["configs"] = config_table(K, max(20, args.steps // 2), args.warmup, args.only)
    if args.torch_native:
        result["torch_native"] = torch_native_table(K, max(20, args.steps // 2), args.warmup)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(host, gpu_out, fb + bb)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result), flush=True)
    if result["cpu_baseline"] and result["cpu_baseline"]["parity"] and \
            not result["cpu_baseline"]["parity"]["ok"]:
        log("PARITY FAILURE:", json.dumps(result["cpu_baseline"]["parity"]))
        sys.exit(1)


if __name__ == "__main__":
    main()
