"""CPU-side checks of the C++ backend layer (libnnabla_hip.so): it loads,
exports the flat C surface, initialises its registries, and refuses contexts
it has no implementation for - all without touching a device."""
import ctypes
import os
import re

import numpy as np
import pytest

from _util import ROOT, load_package

load_package()
from nnabla_ext_cuda_amd import binding as B  # noqa: E402


def declared():
    text = open(os.path.join(ROOT, "include", "nnabla_hip_capi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nnabla_hip_[a-z0-9_]+)\s*\(", text)))


def test_capi_header_binding_and_library_agree():
    syms = declared()
    assert sorted(B.SIGNATURES) == syms
    h = ctypes.CDLL(B.HOST_LIB_PATH)
    for s in syms:
        assert hasattr(h, s), s


def test_init_is_idempotent_and_registers_backend():
    B.init()
    B.init()
    assert B.lib().nnabla_hip_array_classes() == b"HipCachedArray,HipArray"


def test_variable_roundtrip_on_host_float_and_half():
    B.init()
    rng = np.random.default_rng(0)
    a = rng.standard_normal((3, 4, 5)).astype(np.float32)
    v = B.Variable(a.shape)
    assert v.current_shape == (3, 4, 5)
    v.set_data(a)
    np.testing.assert_array_equal(v.d, a)
    v.set_data(a, half=True)                       # stored as float16, read back as float32
    np.testing.assert_array_equal(v.d, a.astype(np.float16).astype(np.float32))
    v.fill_grad(2.5)
    np.testing.assert_array_equal(v.g, np.full(a.shape, 2.5, np.float32))
    v.zero_grad()
    np.testing.assert_array_equal(v.g, np.zeros(a.shape, np.float32))
    with pytest.raises(B.NblaError):
        v.set_data(np.zeros(7, np.float32))        # wrong element count


def test_registry_selects_by_context_and_has_no_cpu_implementation():
    B.init()
    f = B.BatchNormalization(B.context(type_config="float"))
    assert f.name == "BatchNormalizationHip"
    assert B.LayerNormalization(B.context(type_config="half")).name == "LayerNormalizationHip"
    assert B.GroupNormalization(B.context(type_config="float"), num_groups=2).name == "GroupNormalizationHip"
    assert B.InstanceNormalization(B.context(type_config="half")).name == "InstanceNormalizationHip"
    assert B.FusedBatchNormalization(B.context(type_config="half")).name == "FusedBatchNormalizationHip"
    assert B.TensorNormalization(B.context(type_config="float")).name == "TensorNormalizationHip"
    assert B.WeightStandardization(B.context(type_config="half")).name == "WeightStandardizationHip"
    cpu_only = {"backends": "cpu:float", "array_class": "CpuArray", "device_id": "0"}
    for make in (B.BatchNormalization, B.LayerNormalization, B.GroupNormalization,
                 B.InstanceNormalization, B.FusedBatchNormalization, B.TensorNormalization,
                 B.WeightStandardization):
        with pytest.raises(B.NblaError, match="No implementation"):
            make(cpu_only)


def test_setup_rejects_wrong_array_class_before_any_device_work():
    B.init()
    ctx = {"backends": "hip:float", "array_class": "CpuArray", "device_id": "0"}
    f = B.LayerNormalization(ctx)
    x, y = B.Variable((4, 8)), B.Variable((4, 8))
    beta, gamma = B.Variable((1, 8)), B.Variable((1, 8))
    with pytest.raises(B.NblaError, match="not allowed"):
        f.setup([x, beta, gamma], [y])
    f2 = B.LayerNormalization(B.context(type_config="float"))
    with pytest.raises(B.NblaError, match="setup"):
        f2.forward([x, beta, gamma], [y])          # forward before setup


def test_context_follows_the_reference_signature():
    assert B.context() == {"backends": "hip:float", "array_class": "HipCachedArray",
                           "device_id": "0"}
    assert B.context(1, "half")["backends"] == "hip:half,hip:float"
    assert B.context(device_id=3)["device_id"] == "3"
    with pytest.raises(ValueError, match="Unknown data type config"):
        B.context(0, "mixed_half")
    assert B.array_classes() == ["HipCachedArray", "HipArray"]


def test_product_has_no_fallback_and_never_touches_the_oracle(tmp_path):
    """The package raises when its kernel library is missing, and no file of
    the package imports, loads or names the oracle."""
    import importlib.util
    import pathlib
    import re
    root = pathlib.Path(__file__).resolve().parents[1]
    pkg = root / "nnabla-ext-cuda_amd"
    spec = importlib.util.spec_from_file_location("nblahip_missing", pkg / "__init__.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod.LIB_PATH = str(tmp_path / "libnblahip.so")          # not there
    with pytest.raises(RuntimeError, match="no fallback"):
        mod.lib()
    pat = re.compile(r"oracle|norm_ref|libnorm_ref")
    offenders = []
    for f in pkg.rglob("*"):
        if f.is_file() and f.suffix in {".py", ".cpp", ".hpp", ".h", ".hip", ".cuh"} or f.name == "Makefile":
            if f.is_file() and pat.search(f.read_text(errors="ignore")):
                offenders.append(str(f.relative_to(root)))
    assert not offenders, offenders
