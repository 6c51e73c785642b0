"""nblahip_permute against numpy.transpose (bit-exact: it only moves data):
every branch of the kernel pair - same innermost axis (runs), different
innermost axes (LDS tiles), merged and unit axes, ragged tile edges, both
dtypes, accumulation."""
import ctypes

import numpy as np
import pytest

from _util import load_package

K = load_package()

CASES = [
    ((6, 10), (1, 0)),
    ((64, 64), (1, 0)),
    ((65, 130), (1, 0)),
    ((3, 5, 7), (2, 0, 1)),
    ((3, 5, 7), (0, 2, 1)),
    ((3, 5, 7), (1, 0, 2)),            # innermost axis kept: run kernel
    ((4, 6, 8, 10), (0, 2, 3, 1)),     # NCHW -> NHWC
    ((4, 6, 8, 10), (0, 3, 1, 2)),     # NHWC -> NCHW
    ((2, 3, 16, 5, 7), (0, 2, 1, 3, 4)),
    ((2, 3, 16, 5, 7), (4, 3, 2, 1, 0)),
    ((2, 1, 16, 1, 7), (4, 3, 2, 1, 0)),
    ((5, 1, 1), (2, 1, 0)),
    ((7,), (0,)),
    ((2, 70, 3, 129), (0, 3, 2, 1)),
    ((3, 4, 5, 6, 7, 2), (5, 0, 3, 1, 4, 2)),
    ((8, 56, 56, 32), (0, 3, 1, 2)),
    ((2, 2, 2, 2, 2, 2, 2, 2), (7, 6, 5, 4, 3, 2, 1, 0)),
]


@pytest.mark.gpu
@pytest.mark.parametrize("dt", ["f32", "f16"])
@pytest.mark.parametrize("shape,perm", CASES)
def test_permute_matches_numpy(shape, perm, dt):
    import torch
    rng = np.random.default_rng(7)
    npdt = np.float16 if dt == "f16" else np.float32
    a = rng.standard_normal(shape).astype(npdt)
    x = torch.from_numpy(a).cuda()
    y = K.permute(x, perm)
    ref = np.ascontiguousarray(np.transpose(a, perm))
    assert tuple(y.shape) == ref.shape
    assert np.array_equal(y.cpu().numpy(), ref)
    # back again through the inverse permutation
    inv = [0] * len(perm)
    for i, p in enumerate(perm):
        inv[p] = i
    assert np.array_equal(K.permute(y, inv).cpu().numpy(), a)


@pytest.mark.gpu
@pytest.mark.parametrize("shape,perm", [((4, 6, 8, 10), (0, 2, 3, 1)), ((3, 5, 7), (1, 0, 2))])
def test_permute_accumulates(shape, perm):
    import torch
    rng = np.random.default_rng(8)
    a = rng.standard_normal(shape).astype(np.float32)
    b = rng.standard_normal([shape[p] for p in perm]).astype(np.float32)
    out = torch.from_numpy(b).cuda()
    K.permute(torch.from_numpy(a).cuda(), perm, out=out, accum=True)
    assert np.array_equal(out.cpu().numpy(), b + np.transpose(a, perm))


def test_permute_rejects_bad_arguments():
    L = K.lib()
    shape = (ctypes.c_int64 * 3)(2, 3, 4)
    bad = (ctypes.c_int * 3)(0, 0, 1)
    ok = (ctypes.c_int * 3)(2, 0, 1)
    assert L.nblahip_permute(None, None, 3, shape, bad, 0, 0, None) == -1   # not a permutation
    assert L.nblahip_permute(None, None, 3, shape, ok, 0, 0, None) == -1    # null tensors
    assert L.nblahip_permute(None, None, 9, shape, ok, 0, 0, None) == -1    # too many axes
    assert L.nblahip_permute(None, None, 3, shape, ok, 0, 7, None) == -1    # dtype
    empty = (ctypes.c_int64 * 3)(2, 0, 4)
    assert L.nblahip_permute(None, None, 3, empty, ok, 0, 0, None) == 0
    big = (ctypes.c_int64 * 3)(1 << 20, 1 << 10, 4)
    assert L.nblahip_permute(None, None, 3, big, ok, 0, 0, None) == -3
