"""Shared helpers of the test-suite: package loading, tolerances, input
generators for the benchmark configurations."""
import importlib.util
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_DIR = os.path.join(ROOT, "nnabla-ext-cuda_amd")
PKG_NAME = "nnabla_ext_cuda_amd"


def load_package():
    """Import nnabla-ext-cuda_amd/ (the directory name is not an identifier)."""
    if PKG_NAME in sys.modules:
        return sys.modules[PKG_NAME]
    spec = importlib.util.spec_from_file_location(
        PKG_NAME, os.path.join(PKG_DIR, "__init__.py"), submodule_search_locations=[PKG_DIR])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[PKG_NAME] = mod
    spec.loader.exec_module(mod)
    return mod


# Tolerances stated by the task: fp32 rel <= 1e-5 / abs <= 1e-5 on y, mean/var
# and gradients; fp16 rel <= 2e-3 on y and <= 1e-2 on gradients (statistics are
# float32 in either mode).  Kinds:
#   y, stat, grad : elementwise tensors; the absolute floor is 1e-5 in fp32
#                   (as stated) and rtol * RMS(reference) in fp16 (no absolute
#                   figure is stated, so the floor follows the tensor's scale);
#   pgrad         : dgamma/dbeta, sums of up to 10^6 terms: the floor is
#                   relative to the RMS over the vector, because the rounding
#                   error of a sum follows the size of its terms, not of the
#                   (possibly cancelling) result.
TOL = {
    ("f32", "y"): (1e-5, 1e-5),
    ("f32", "stat"): (1e-5, 1e-5),
    ("f32", "grad"): (1e-5, 1e-5),
    ("f32", "pgrad"): (1e-5, 1e-5),
    ("f16", "y"): (2e-3, 2e-3),
    ("f16", "stat"): (1e-5, 1e-5),
    ("f16", "grad"): (1e-2, 1e-2),
    ("f16", "pgrad"): (1e-2, 1e-2),
}


def assert_close(got, ref, dtype, kind, name="", scale=None):
    """|got - ref| <= atol*scale + rtol*|ref| elementwise."""
    rtol, atol = TOL[(dtype, kind)]
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    ref = np.asarray(ref, dtype=np.float64).reshape(-1)
    assert got.shape == ref.shape, f"{name}: shape {got.shape} vs {ref.shape}"
    if got.size == 0:
        return
    assert np.isfinite(got).all(), f"{name}: non-finite values in the result"
    if scale is None:
        rms = float(np.sqrt(np.mean(ref * ref)))
        if kind == "pgrad":
            scale = max(1.0, rms)
        elif dtype == "f16" and kind != "stat":
            scale = rms
        else:
            scale = 1.0
    err = np.abs(got - ref)
    bound = atol * scale + rtol * np.abs(ref)
    bad = err > bound
    if bad.any():
        i = int(np.argmax(err - bound))
        raise AssertionError(
            f"{name}: {int(bad.sum())}/{got.size} outside tolerance "
            f"(rtol={rtol}, atol={atol}*{scale:.3g}); worst at {i}: got {got[i]!r} "
            f"ref {ref[i]!r} err {err[i]:.3e} bound {bound[i]:.3e}")


def dtype_name(t):
    import torch
    return "f16" if t == torch.float16 else "f32"


def to_dev(a, dtype=None):
    """numpy -> cuda tensor (float32 unless dtype given)."""
    import torch
    if a is None:
        return None
    t = torch.from_numpy(np.ascontiguousarray(a))
    t = t.to(dtype if dtype is not None else torch.float32)
    return t.cuda()


def to_np(t):
    return None if t is None else t.detach().float().cpu().numpy().astype(np.float64)


def rounded(a, dtype):
    """The values a tensor of `dtype` actually holds, as float64."""
    import torch
    if dtype == torch.float16:
        return np.asarray(a, dtype=np.float16).astype(np.float64)
    return np.asarray(a, dtype=np.float32).astype(np.float64)
