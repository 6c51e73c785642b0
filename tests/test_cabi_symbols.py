"""CPU-side checks of the C-ABI library: it loads without a GPU, exports
every symbol include/nblahip.h declares, and its host-only entry points
(status text, workspace sizing, argument validation) behave."""
import ctypes
import os
import re

from _util import ROOT, load_package

K = load_package()


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "nblahip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nblahip_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    syms = declared_symbols()
    assert len(syms) >= 25
    assert sorted(K.SIGNATURES) == syms


def test_library_exports_every_declared_symbol():
    handle = ctypes.CDLL(K.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(handle, name), name


def test_status_strings_and_version():
    L = K.lib()
    assert L.nblahip_abi_version() == 1
    assert L.nblahip_error_string(0) == b"success"
    for code in (-1, -2, -3, -4):
        assert b"nblahip" in L.nblahip_error_string(code)


def test_workspace_sizes_are_sane():
    L = K.lib()
    # BN config 2 and 5: partials + per-channel parameters, well under 16 MiB
    for args in ((32, 256, 3136, 0), (802816, 64, 1, 1)):
        n = L.nblahip_bn_workspace_bytes(*args)
        assert 0 < n < (16 << 20) and n % 256 == 0
    n = L.nblahip_ln_bwd_workspace_bytes(16384, 1024, 0)
    assert 0 < n < (64 << 20)
    assert L.nblahip_gn_bwd_workspace_bytes(16, 256, 4096, 32, 1) >= 16 * 256 * 8
    assert L.nblahip_in_bwd_workspace_bytes(16, 256, 4096, 1) >= 16 * 256 * 8
    # invalid shapes size to 0
    assert L.nblahip_bn_workspace_bytes(-1, 4, 4, 0) == 0
    assert L.nblahip_gn_bwd_workspace_bytes(2, 6, 4, 4, 0) == 0


def test_argument_validation_needs_no_gpu():
    L = K.lib()
    # rejected before anything touches the device
    assert L.nblahip_ln_fwd(None, None, None, None, None, None, 4, 4, 1e-5, 0, None) == -1
    assert L.nblahip_bn_fwd_infer(None, None, None, None, None, None, 4, 4, 4, 1e-5, 9, None) == -1
    assert L.nblahip_ln_fwd(None, None, None, None, None, None, 0, 4, 1e-5, 0, None) == 0
    assert L.nblahip_convert(None, 0, None, 1, 0, None) == 0


def test_row_forwards_reject_an_output_that_overlaps_an_input():
    """y may be x itself; any other overlap with x, the parameters or the
    statistics is refused from the pointer ranges alone (no device access)."""
    L = K.lib()
    base = 0x7f0000000000                      # never dereferenced
    n_ln, r_ln = 64, 256                       # fp32: 65536 bytes
    x, far = base, base + (1 << 24)
    g, b, m, v = far, far + 4096, far + 8192, far + 12288

    def ln(y, gamma=g, beta=b, mean=m, var=v):
        return L.nblahip_ln_fwd(x, gamma, beta, y, mean, var, n_ln, r_ln, 1e-5, 0, None)

    assert ln(x + 1024) == -4 and ln(x - 1024) == -4 and ln(x + 65532) == -4
    assert ln(far - 32768, gamma=far) == -4     # y runs into gamma
    assert ln(x + (1 << 20), mean=x + (1 << 20) + 100) == -4
    assert "overlaps" in L.nblahip_error_string(-4).decode()
    gn = lambda y: L.nblahip_gn_fwd(x, g, b, y, m, v, 4, 16, 64, 4, 1e-5, 1, None)   # fp16: 8192 bytes
    assert gn(x + 4096) == -4 and gn(x - 8190) == -4
    inn = lambda y, beta=b: L.nblahip_in_fwd(x, g, beta, y, m, v, 4, 16, 64, 1, 0, 1e-5, 1, None)
    assert inn(x + 2) == -4
    assert inn(far + 4096 - 8192 + 4 * 16 * 4, beta=b) == -4   # per-sample beta: 4*16 floats
