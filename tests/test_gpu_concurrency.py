"""The C-ABI under the calling patterns of a framework: many host threads, each
on its own stream (the reference trains from several threads at once,
src/nbla/cuda/test/test_multi_thread_training.cpp:153-198), and capture into a
graph that is replayed (no entry point allocates, synchronises or clears
memory behind the caller's back)."""
import threading

import numpy as np
import pytest
import torch

from _util import load_package

pytestmark = pytest.mark.gpu
K = load_package()


def _work(kind, seed, dtype):
    """One forward+backward of a normalization on tensors derived from seed;
    returns every output."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    if kind == "bn":
        x = (torch.randn(16, 32, 14, 14, device="cuda", generator=g) * 2 + 1).to(dtype)
        dy = torch.randn(16, 32, 14, 14, device="cuda", generator=g).to(dtype)
        gamma = torch.rand(32, device="cuda", generator=g) + 0.5
        beta = torch.randn(32, device="cuda", generator=g)
        rm, rv = torch.zeros(32, device="cuda"), torch.ones(32, device="cuda")
        y, m, v = K.bn_forward_batch(x, beta, gamma, rm, rv, 1, 0.9, 1e-5)
        dx, dg, db = K.bn_backward(x, dy, gamma, m, v, 1, 1e-5)
        return [y, m, v, rm, rv, dx, dg, db]
    if kind == "bn_cl":
        x = torch.randn(8, 14, 14, 64, device="cuda", generator=g).to(dtype)
        dy = torch.randn(8, 14, 14, 64, device="cuda", generator=g).to(dtype)
        gamma = torch.rand(64, device="cuda", generator=g) + 0.5
        beta = torch.randn(64, device="cuda", generator=g)
        z = torch.randn(8, 14, 14, 64, device="cuda", generator=g).to(dtype)
        y, m, v = K.fused_bn_forward_batch(x, z, beta, gamma, None, None, 3, 0.9, 1e-5)
        dx, dz, dg, db = K.fused_bn_backward(x, y, dy, gamma, m, v, 3, 1e-5)
        return [y, m, v, dx, dz, dg, db]
    if kind == "ln":
        x = torch.randn(256, 768, device="cuda", generator=g).to(dtype)
        dy = torch.randn(256, 768, device="cuda", generator=g).to(dtype)
        gamma = torch.rand(768, device="cuda", generator=g) + 0.5
        beta = torch.randn(768, device="cuda", generator=g)
        y, m, v = K.ln_forward(x, beta, gamma, 256, 1e-5)
        dx, dg, db = K.ln_backward(x, dy, gamma, m, v, 256, 1e-5)
        return [y, m, v, dx, dg, db]
    if kind == "gn":
        x = torch.randn(4, 32, 16, 16, device="cuda", generator=g).to(dtype)
        dy = torch.randn(4, 32, 16, 16, device="cuda", generator=g).to(dtype)
        gamma = torch.rand(32, device="cuda", generator=g) + 0.5
        beta = torch.randn(32, device="cuda", generator=g)
        y, m, v = K.gn_forward(x, beta, gamma, 8, 1e-5)
        dx, dg, db = K.gn_backward(x, dy, gamma, m, v, 8, 1e-5)
        return [y, m, v, dx, dg, db]
    x = torch.randn(4, 12, 12, 32, device="cuda", generator=g).to(dtype)
    dy = torch.randn(4, 12, 12, 32, device="cuda", generator=g).to(dtype)
    gamma = torch.rand(32, device="cuda", generator=g) + 0.5
    beta = torch.randn(32, device="cuda", generator=g)
    y, m, v = K.in_forward(x, beta, gamma, 1e-5, channel_last=True)
    dx, dg, db = K.in_backward(x, dy, gamma, m, v, 1e-5, channel_last=True)
    return [y, m, v, dx, dg, db]


KINDS = ["bn", "bn_cl", "ln", "gn", "in_cl"]


def test_many_threads_on_their_own_streams():
    jobs = [(k, 100 + i, dt) for i, k in enumerate(KINDS)
            for dt in (torch.float32, torch.float16)]
    want = [[t.clone() for t in _work(*j)] for j in jobs]
    torch.cuda.synchronize()
    got = [None] * len(jobs)
    errors = []

    def run(i):
        try:
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                for _ in range(5):                      # repeated: same answer every time
                    out = _work(*jobs[i])
                s.synchronize()
            got[i] = out
        except Exception as e:  # noqa: BLE001 - reported below
            errors.append((jobs[i], repr(e)))

    threads = [threading.Thread(target=run, args=(i,)) for i in range(len(jobs))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for j, w, g_ in zip(jobs, want, got):
        for a, b in zip(w, g_):
            assert torch.equal(a, b), j


@pytest.mark.parametrize("kind", KINDS)
def test_graph_capture_and_replay(kind):
    """Capture forward+backward, replay three times with new inputs in the
    captured buffers and eager work in between; every replay equals eager."""
    L = K.lib()
    dtype = torch.float16
    st = torch.cuda.Stream()
    shape = {"bn": (16, 32, 14, 14), "bn_cl": (8, 14, 14, 64), "ln": (256, 768),
             "gn": (4, 32, 16, 16), "in_cl": (4, 12, 12, 32)}[kind]
    c = {"bn": 32, "bn_cl": 64, "ln": 768, "gn": 32, "in_cl": 32}[kind]
    x = torch.empty(shape, device="cuda", dtype=dtype)
    dy = torch.empty_like(x)
    gamma = torch.rand(c, device="cuda") + 0.5
    beta = torch.randn(c, device="cuda")

    def eager(xi, dyi):
        if kind == "bn":
            y, m, v = K.bn_forward_batch(xi, beta, gamma, None, None, 1, 0.9, 1e-5)
            return [y, m, v, *K.bn_backward(xi, dyi, gamma, m, v, 1, 1e-5)]
        if kind == "bn_cl":
            y, m, v = K.fused_bn_forward_batch(xi, None, beta, gamma, None, None, 3, 0.9, 1e-5)
            return [y, m, v, *K.fused_bn_backward(xi, y, dyi, gamma, m, v, 3, 1e-5)]
        if kind == "ln":
            y, m, v = K.ln_forward(xi, beta, gamma, shape[0], 1e-5)
            return [y, m, v, *K.ln_backward(xi, dyi, gamma, m, v, shape[0], 1e-5)]
        if kind == "gn":
            y, m, v = K.gn_forward(xi, beta, gamma, 8, 1e-5)
            return [y, m, v, *K.gn_backward(xi, dyi, gamma, m, v, 8, 1e-5)]
        y, m, v = K.in_forward(xi, beta, gamma, 1e-5, channel_last=True)
        return [y, m, v, *K.in_backward(xi, dyi, gamma, m, v, 1e-5, channel_last=True)]

    x.normal_()
    dy.normal_()
    eager(x, dy)                                   # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(st):
        with torch.cuda.graph(graph, stream=st):
            outs = eager(x, dy)
    torch.cuda.synchronize()
    for rep in range(3):
        xi = torch.randn(shape, device="cuda").to(dtype) * (rep + 1)
        dyi = torch.randn(shape, device="cuda").to(dtype)
        want = [t.clone() for t in eager(xi, dyi)]
        x.copy_(xi)
        dy.copy_(dyi)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(want, outs):
            assert torch.equal(a, b), (kind, rep)
    assert L.nblahip_abi_version() >= 1
