"""Host side of the plan knobs (no GPU): the override order of
nblahip_tune_set / environment / default, and that every knob the kernel
sources read has a parity case in tests/test_gpu_plan_knobs.py."""
import os
import re
import subprocess
import sys

import pytest

from _util import ROOT, load_package

K = load_package()


def test_every_knob_the_library_reads_has_a_parity_case():
    import test_gpu_plan_knobs as T
    src = os.path.join(K.CSRC, "kernels")
    read = set()
    for fn in os.listdir(src):
        text = open(os.path.join(src, fn)).read()
        read |= set(re.findall(r'tune_int\("([A-Z0-9_]+)"', text))
    used = set()
    for case in T.SWITCHES:
        used |= set(case[3])
        if len(case) > 6:
            used |= set(case[6])
    for case in T.GRIDS:
        for knobs in case[3]:
            used |= set(knobs)
    assert len(read) >= 30
    assert read == used, f"no parity case: {sorted(read - used)}; unknown: {sorted(used - read)}"


def test_override_order_and_reset():
    env = {k: v for k, v in os.environ.items() if not k.startswith("NBLAHIP_")}
    env["NBLAHIP_BN_ROWS"] = "0"
    env["NBLAHIP_ROW_TPR"] = "junk"
    code = """
import sys
sys.path.insert(0, %r)
from _util import load_package
K = load_package()
assert K.tune_get("BN_ONCHIP", 7) == 7          # default: the caller's fallback
assert K.tune_get("BN_ROWS", 1) == 0            # environment over default
assert K.tune_get("ROW_TPR", 5) == 5            # unparsable: ignored
K.tune_set("BN_ROWS", 2)
K.tune_set("BN_ONCHIP", 0)
assert K.tune_get("BN_ROWS", 1) == 2            # set over environment
assert K.tune_get("BN_ONCHIP", 7) == 0
K.tune_set("BN_ROWS", -1)
assert K.tune_get("BN_ROWS", 1) == 0            # undone: environment again
K.tune_reset()
assert K.tune_get("BN_ONCHIP", 7) == 7
L = K.lib()
assert L.nblahip_tune_set(None, 1) == -1
assert L.nblahip_tune_set(b"", 1) == -1
assert L.nblahip_tune_set(b"BN_ROWS", 1 << 20) == -1
print("ok")
""" % os.path.join(ROOT, "tests")
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True,
                         timeout=120)
    assert out.returncode == 0 and out.stdout.strip() == "ok", out.stdout + out.stderr


def test_profile_kernel_list_is_empty_without_launches():
    assert K.profile_kernels() == []
