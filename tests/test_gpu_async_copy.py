"""Asynchronous host<->device copies of the array layer (the reference's
AsyncFlag::ASYNC / UNSAFE synchronizers, src/nbla/cuda/array/cuda_array.cpp:
83-158): enqueued on the backend's transfer streams for page-locked host
arrays, ordered against the function stream by events, blocking for pageable
memory.  Every case checks the data that arrives, through a Function or a
read-back."""
import numpy as np
import pytest

from _util import assert_close, load_package
from oracle import norm_ref as R

load_package()
from nnabla_ext_cuda_amd import binding as B  # noqa: E402

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _host_class():
    B.init()
    yield
    B.set_host_array_class("CpuArray")
    B.device_synchronize()


def _ln(x_var, shape, outer):
    f = B.LayerNormalization(B.context(), batch_axis=[0], eps=1e-5, no_scale=True, no_bias=True)
    y = B.Variable(shape)
    f.setup([x_var], [y])
    f.forward([x_var], [y])
    return y


@pytest.mark.parametrize("host_class", ["HipCachedHostArray", "CpuArray"])
@pytest.mark.parametrize("flags", [B.ASYNC, B.ASYNC | B.UNSAFE, 0])
def test_async_upload_feeds_a_function_and_async_download_returns_its_output(host_class, flags):
    B.set_host_array_class(host_class)
    rng = np.random.default_rng(41)
    shape = (512, 1024)
    x = rng.standard_normal(shape).astype(np.float32) + 2
    vx = B.Variable(shape)
    vx.set_data(x)                                   # lives in a host array of host_class
    vx.cast("HipCachedArray", async_flags=flags)     # upload, enqueued when pinned + ASYNC
    vy = _ln(vx, shape, shape[0])                    # the kernel's stream waits for the upload
    y_r, _, _ = R.ln_forward(x, None, None, shape[0], 1e-5)
    vy.cast(host_class, device_id="", async_flags=flags)   # download, enqueued likewise
    assert_close(vy.d, y_r, "f32", "y", "y after asynchronous transfers")  # the host waits here
    B.device_synchronize()
    assert B.pending_transfers() == 0


def test_source_of_an_async_upload_outlives_its_variable_slot():
    """The upload drops the host array from the variable at once; its memory
    must stay valid until the copy has run even when new page-locked arrays are
    allocated and filled right behind it."""
    B.set_host_array_class("HipCachedHostArray")
    n = 16 << 20
    x = np.arange(n, dtype=np.float32)
    vx = B.Variable((n,))
    vx.set_data(x)
    vx.cast("HipCachedArray", async_flags=B.ASYNC)
    others = []
    for k in range(3):                               # same size: likely the same pages again
        v = B.Variable((n,))
        v.set_data(np.full(n, -1.0 - k, np.float32))
        others.append(v)
    assert B.pending_transfers() <= 1
    np.testing.assert_array_equal(vx.d, x)
    B.device_synchronize()
    assert B.pending_transfers() == 0


def test_unsafe_upload_keeps_no_guard():
    B.set_host_array_class("HipCachedHostArray")
    x = np.linspace(-1, 1, 4096, dtype=np.float32)
    vx = B.Variable((4096,))
    vx.set_data(x)
    vx.cast("HipCachedArray", async_flags=B.ASYNC | B.UNSAFE)
    assert B.pending_transfers() == 0
    B.device_synchronize()
    np.testing.assert_array_equal(vx.d, x)


def test_half_storage_goes_through_the_same_path():
    B.set_host_array_class("HipCachedHostArray")
    x = np.linspace(-4, 4, 8192, dtype=np.float32)
    vx = B.Variable((8192,))
    vx.set_data(x, half=True)
    vx.cast("HipCachedArray", half=True, async_flags=B.ASYNC)
    vx.cast("HipCachedArray", half=False)            # device-side conversion after the upload
    np.testing.assert_array_equal(vx.d, x.astype(np.float16).astype(np.float32))


@pytest.mark.parametrize("dtype", ["int32", "uint8", "int64", "bool", "float64"])
def test_device_arrays_store_every_dtype(dtype):
    """Stored and copied without conversion, host -> device -> host, also
    through the asynchronous path; zero() clears them."""
    B.set_host_array_class("HipCachedHostArray")
    rng = np.random.default_rng(5)
    a = (rng.integers(0, 200, 5000) % (2 if dtype == "bool" else 200)).astype(dtype)
    v = B.Variable((5000,))
    v.set_raw(a)
    v.cast_raw("HipCachedArray", dtype, async_flags=B.ASYNC)
    np.testing.assert_array_equal(v.get_raw(dtype), a)
    v.cast_raw("HipArray", dtype)
    v.zero_data()
    np.testing.assert_array_equal(v.get_raw(dtype), np.zeros(5000, dtype))


@pytest.mark.parametrize("dtype,value", [("int8", -5), ("uint8", 200), ("int16", -1234), ("uint16", 60000),
                                         ("int32", 70000), ("uint32", 3000000000), ("int64", -7),
                                         ("uint64", 9), ("bool", 1), ("float64", 2.5),
                                         ("float32", 1.25), ("float16", -0.5)])
def test_device_arrays_fill_every_dtype(dtype, value):
    """fill() with a value other than zero on a device array of any dtype (the
    value converted to the element type), first materialised on the device."""
    v = B.Variable((4099,))
    v.fill_data(value)
    v.cast_raw("HipArray", dtype)
    np.testing.assert_array_equal(v.get_raw(dtype), np.full(4099, value, dtype))


def test_fill_bytes_entry_point():
    """The C-ABI fill of 1-, 2-, 4- and 8-byte elements; an odd element size and
    a misaligned destination are argument errors."""
    import torch
    from _util import load_package
    K = load_package()
    L = K.lib()
    for dt, nbytes, pattern in [(torch.uint8, 1, 0xAB), (torch.int16, 2, 0x1234),
                                (torch.int32, 4, 0x7EADBEEF), (torch.int64, 8, 0x0123456789ABCDEF)]:
        t = torch.zeros(100003, dtype=dt, device="cuda")
        K.check(L.nblahip_fill_bytes(t.data_ptr(), nbytes, pattern, t.numel() - 3, None))
        torch.cuda.synchronize()
        assert (t[:-3] == pattern).all() and (t[-3:] == 0).all()
    t = torch.zeros(64, dtype=torch.int32, device="cuda")
    assert L.nblahip_fill_bytes(t.data_ptr(), 3, 1, 4, None) == -1
    assert L.nblahip_fill_bytes(t.data_ptr() + 2, 4, 1, 4, None) == -1
    assert L.nblahip_fill_bytes(t.data_ptr(), 4, 1, 0, None) == 0


def test_host_reader_of_a_pinned_array_waits_for_its_pending_download():
    """An ASYNC device-to-pinned-host cast leaves the transfer's event on the
    pinned array; a following host read through another host class (a plain
    copy between two host arrays) must wait for it before it copies."""
    n = 32 << 20
    x = np.arange(n, dtype=np.float32)
    vx = B.Variable((n,))
    vx.set_data(x)
    vx.cast("HipCachedArray")
    for k in range(3):
        vx.cast("HipCachedHostArray", device_id="", async_flags=B.ASYNC)   # enqueued, not waited for
        got = vx.d                                                          # CpuArray <- pinned array
        np.testing.assert_array_equal(got, x)
        vx.cast("HipCachedArray")                                           # head back on the device
        x = x + 1
        vx.set_data(x)
        vx.cast("HipCachedArray")
    B.device_synchronize()
    assert B.pending_transfers() == 0
