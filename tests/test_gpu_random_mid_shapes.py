"""Randomly drawn tensors of 2 - 40 MB (fixed seeds), the sizes at which the
plans switch from single launches to the kernels that hold a tensor on the
chip, exchange partial sums or run three launches: forward + backward of
BatchNormalization, LayerNormalization, GroupNormalization and
InstanceNormalization in both layouts against the oracle, channel counts and
planes on and off the 16-byte and 128-byte grids."""
import numpy as np
import pytest
import torch

import test_gpu_plan_knobs as P

pytestmark = pytest.mark.gpu
F32, F16 = torch.float32, torch.float16
CL_CHANNELS = [24, 40, 64, 72, 96, 100, 120, 128, 160, 200, 240, 256, 320, 400, 520, 1000]
CF_CHANNELS = [3, 8, 16, 24, 32, 48, 64, 96, 128, 192, 256, 320, 384, 512, 640, 768, 1024, 1280, 2048]
CF_PLANES = [7, 8, 14, 16, 17, 28, 32, 35, 56, 63, 64, 71, 96, 112, 128]
LN_HIDDEN = [64, 128, 256, 512, 768, 1024, 1023, 1028, 2048, 3072, 4096, 5120, 8192, 12288, 16384]


def divisors(c):
    return [d for d in range(1, c + 1) if c % d == 0]


def log_uniform(rng, lo, hi):
    return int(np.exp(rng.uniform(np.log(lo), np.log(hi))))


@pytest.fixture(autouse=True)
def _default_knobs():
    P.K.tune_reset()
    yield
    P.K.tune_reset()


@pytest.mark.parametrize("seed", range(16))
@pytest.mark.parametrize("kind", ["bn", "gn", "in"])
@pytest.mark.parametrize("channel_last", [False, True], ids=["planes", "channel_last"])
def test_random_mid_size_channels(seed, kind, channel_last):
    rng = np.random.default_rng(7000 + 97 * seed + 13 * ["bn", "gn", "in"].index(kind) + channel_last)
    dtype = F16 if rng.integers(0, 2) else F32
    esz = 2 if dtype == F16 else 4
    target = log_uniform(rng, 2e6, 40e6 if not channel_last else 28e6)
    if channel_last:
        c = int(rng.choice(CL_CHANNELS))
        h = int(rng.integers(12, 80))
        w = h if rng.integers(0, 3) else int(rng.integers(12, 80))
    else:
        c = int(rng.choice(CF_CHANNELS))
        h = int(rng.choice(CF_PLANES))
        w = h if rng.integers(0, 4) else int(rng.integers(5, 100))
    n = max(1, min(256, target // (h * w * c * esz)))
    case_seed = int(rng.integers(0, 1 << 30))
    if kind == "gn":
        P.run_gn(n, c, (h, w), int(rng.choice(divisors(c))), dtype, channel_last, case_seed)
    elif kind == "in":
        P.run_in(n, c, (h, w), dtype, channel_last, case_seed)
    elif channel_last:
        P.run_bn((n, h, w, c), 3, dtype, case_seed)
    else:
        P.run_bn((n, c, h, w), 1, dtype, case_seed)


@pytest.mark.parametrize("seed", range(24))
def test_random_mid_size_rows(seed):
    rng = np.random.default_rng(9000 + seed)
    dtype = F16 if rng.integers(0, 2) else F32
    esz = 2 if dtype == F16 else 4
    hidden = int(rng.choice(LN_HIDDEN)) if seed % 2 else log_uniform(rng, 48, 20000)
    outer = max(1, log_uniform(rng, 2e6, 40e6) // (hidden * esz))
    P.run_ln(outer, hidden, dtype, int(rng.integers(0, 1 << 30)))
