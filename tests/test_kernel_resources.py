"""Register, scratch and LDS budgets of the compiled kernels (no GPU).

The build writes the compiler's resource-usage remarks of every kernel to
nnabla-ext-cuda_amd/lib/resources/<unit>.txt.  Several kernel families here
only pay off while a reduction unit stays in registers and LDS (the on-chip
BatchNormalization, the GN/IN rows held on one CU, the channel-last wide
kernels) and their sources steer the register allocator by hand, so a
toolchain change could bring scratch spills back without any test of results
noticing.  This file holds every kernel to:
  * no scratch at all, except the kernels listed (with their bytes per lane)
    in tests/golden/kernel_scratch_allowance.txt, which may not grow;
  * the families named below spill-free without exception;
  * at most 160 KB of LDS per block and no more vector registers than a
    block of its size can be given on a CU (512 per SIMD lane shared by the
    block's waves).
Regenerate the allowance file after a deliberate change with
  python tests/test_kernel_resources.py --write-allowance
"""
import os
import re
import subprocess
import sys

import pytest

from _util import ROOT, load_package

K = load_package()
RES_DIR = os.path.join(os.path.dirname(K.LIB_PATH), "resources")
ALLOWANCE = os.path.join(ROOT, "tests", "golden", "kernel_scratch_allowance.txt")
LDS_PER_CU = 160 * 1024

# Families that must never spill: a spill there turns the on-chip plan into
# extra memory traffic, which is all these kernels exist to avoid.  The second
# field excludes instantiations that are known to spill and are dispatched only
# where they still win (listed in the allowance file).
SPILL_FREE = [
    (r"bn_onchip_fwd_kernel", None),
    (r"bn_onchip_bwd_kernel", r"Li24ELi16ELi8ELi512E"),   # 24 + 16 slots, 512 threads
    (r"row_onchip_fwd_kernel", None),
    (r"gn_cl_wide_fwd_kernel", None),
    (r"in_cl_wide_fwd_kernel", None),
    (r"gn_cl_row_fwd_kernel", None),
    (r"gn_cl_row_bwd_kernel", None),
    (r"bn_stats_\w+_kernel", None),
    (r"bn_apply_\w+_kernel", None),
    (r"bn_bwd_reduce_\w+_kernel", None),
    (r"bn_bwd_apply_\w+_kernel", None),
]


def read_resources():
    if not os.path.isdir(RES_DIR):
        pytest.fail(f"{RES_DIR} is missing: build with make -C {K.CSRC} (it writes the files)")
    out = {}
    for fn in sorted(os.listdir(RES_DIR)):
        for line in open(os.path.join(RES_DIR, fn)):
            parts = line.split()
            if not parts:
                continue
            out[parts[0]] = {k: int(v) for k, v in (p.split("=") for p in parts[1:])}
    return out


def read_allowance():
    allow = {}
    for line in open(ALLOWANCE):
        if line.strip() and not line.startswith("#"):
            name, nbytes = line.split()
            allow[name] = int(nbytes)
    return allow


def block_threads(name):
    """Threads per block of an instantiation whose template carries it (the
    row kernels: <T, VEC, NL, TPR, ...>; the on-chip kernels: <..., THREADS, ...>)."""
    m = re.search(r"(?:row_fwd_kernel|row_bwd_kernel)I(?:f|6__half)Li\d+ELi\d+ELi(\d+)E", name)
    if m:
        return max(int(m.group(1)), 64)
    m = re.search(r"bn_onchip_bwd_kernelI(?:f|6__half)Li\d+ELi\d+ELi\d+ELi\d+ELi(\d+)E", name)
    if m:
        return int(m.group(1))
    return None


def test_resource_files_cover_the_library():
    res = read_resources()
    assert len(res) > 1000
    for family in ("bn_onchip_fwd_kernel", "bn_onchip_bwd_kernel", "row_onchip_fwd_kernel",
                   "cl_wide_bwd_kernel", "gn_cl_wide_fwd_kernel", "in_cl_wide_fwd_kernel",
                   "row_fwd_kernel", "row_bwd_kernel", "permute_tile_kernel"):
        assert any(family in n for n in res), family


def test_no_kernel_spills_beyond_its_allowance():
    res, allow = read_resources(), read_allowance()
    grown = {n: (r["scratch"], allow.get(n, 0)) for n, r in res.items()
             if r["scratch"] > allow.get(n, 0)}
    assert not grown, "scratch bytes per lane (now, allowed): " + repr(grown)
    stale = sorted(n for n in allow if n not in res)
    assert not stale, f"allowance names kernels the library no longer has: {stale}"


def test_on_chip_families_are_spill_free():
    res = read_resources()
    for family, excluded in SPILL_FREE:
        names = [n for n in res if re.search(r"\d+" + family + r"I", n)
                 and not (excluded and re.search(excluded, n))]
        assert names, family
        bad = {n: res[n]["scratch"] for n in names if res[n]["scratch"]}
        assert not bad, f"{family}: {bad}"


def test_lds_and_register_ceilings():
    res = read_resources()
    for name, r in res.items():
        assert r["lds"] <= LDS_PER_CU, (name, r)
        t = block_threads(name)
        if t:   # accumulation registers count against the same file
            assert r["vgpr"] + r["agpr"] <= 512 // max(1, t // 256), (name, r)
    # the layouts that fill a CU: 1024 threads may use 128 registers each
    full = [r for n, r in res.items() if "bn_onchip_fwd_kernel" in n or "row_onchip_fwd_kernel" in n]
    assert full and all(r["vgpr"] <= 128 and r["agpr"] == 0 for r in full)


if __name__ == "__main__":
    if "--write-allowance" in sys.argv:
        rows = sorted((n, r["scratch"]) for n, r in read_resources().items() if r["scratch"])
        with open(ALLOWANCE, "w") as f:
            f.write("# <mangled kernel name> <scratch bytes per lane the build may use>\n")
            for n, b in rows:
                f.write(f"{n} {b}\n")
        print(f"wrote {len(rows)} kernels to {ALLOWANCE}")
