"""Runs the C++ unit test of the host layer (tests/cpp/host_layer_test.cpp),
built with AddressSanitizer and UBSan, leak detection on.  Host code only: no
GPU is needed."""
import os
import pathlib
import subprocess

ROOT = pathlib.Path(__file__).resolve().parents[1]
CSRC = ROOT / "nnabla-ext-cuda_amd" / "csrc"
BIN = CSRC / "build" / "host_layer_test"


def test_host_layer_under_asan_and_ubsan():
    build = subprocess.run(["make", "-C", str(CSRC), "-j8", "host_test"], capture_output=True,
                           text=True)
    assert build.returncode == 0, build.stdout[-3000:] + build.stderr[-3000:]
    env = dict(os.environ,
               ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:verify_asan_link_order=0",
               UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    run = subprocess.run([str(BIN)], capture_output=True, text=True, env=env, timeout=120)
    out = run.stdout + run.stderr
    assert run.returncode == 0, out[-4000:]
    assert " 0 failed" in run.stdout, out[-4000:]
    assert "ERROR: AddressSanitizer" not in out and "runtime error:" not in out, out[-4000:]
    assert "LeakSanitizer" not in out, out[-4000:]
