"""ctypes binding of libnnabla_hip.so (include/nnabla_hip_capi.h): the C++
backend layer - context-selected nbla::Function objects over Variables - as a
language binding sees it.  Used by the tests that exercise the Function
classes the way NNabla's own function tests do (create by name and context,
setup, forward, backward with propagate_down/accum)."""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
HOST_LIB_PATH = os.path.join(_HERE, "lib", "libnnabla_hip.so")

_P = ctypes.c_void_p
_PP = ctypes.POINTER(ctypes.c_void_p)
_I = ctypes.c_int
_I64 = ctypes.c_int64
_F = ctypes.c_float
_S = ctypes.c_char_p
_IP = ctypes.POINTER(ctypes.c_int)
_FP = ctypes.POINTER(ctypes.c_float)

SIGNATURES = {
    "nnabla_hip_init": (_I, []),
    "nnabla_hip_last_error": (_S, []),
    "nnabla_hip_array_classes": (_S, []),
    "nnabla_hip_device_synchronize": (_I, [_S]),
    "nnabla_hip_set_host_array_class": (_I, [_S]),
    "nnabla_hip_device_count": (_I, [ctypes.POINTER(ctypes.c_int)]),
    "nnabla_hip_memory_stats": (_I, [ctypes.POINTER(ctypes.c_uint64)] * 2),
    "nnabla_hip_clear_memory_cache": (_I, []),
    "nnabla_hip_variable_new": (_P, [_I, ctypes.POINTER(_I64)]),
    "nnabla_hip_variable_delete": (None, [_P]),
    "nnabla_hip_variable_ndim": (_I, [_P]),
    "nnabla_hip_variable_shape": (_I, [_P, ctypes.POINTER(_I64)]),
    "nnabla_hip_variable_set": (_I, [_P, _I, _FP, _I64, _I]),
    "nnabla_hip_variable_get": (_I, [_P, _I, _FP, _I64]),
    "nnabla_hip_variable_cast": (_I, [_P, _I, _S, _S, _I, _I, _I]),
    "nnabla_hip_variable_set_raw": (_I, [_P, _I, ctypes.c_void_p, _I64, _I]),
    "nnabla_hip_variable_get_raw": (_I, [_P, _I, ctypes.c_void_p, _I64, _I]),
    "nnabla_hip_pending_transfers": (_I, [ctypes.POINTER(ctypes.c_uint64)]),
    "nnabla_hip_variable_zero": (_I, [_P, _I]),
    "nnabla_hip_variable_fill": (_I, [_P, _I, _F]),
    "nnabla_hip_variable_stored_dtype": (_I, [_P, _I, ctypes.POINTER(_I)]),
    "nnabla_hip_create_batch_normalization": (_P, [_S, _S, _S, _IP, _I, _F, _F, _I, _I, _I]),
    "nnabla_hip_create_fused_batch_normalization": (_P, [_S, _S, _S, _IP, _I, _F, _F, _I, _S]),
    "nnabla_hip_create_layer_normalization": (_P, [_S, _S, _S, _IP, _I, _F, _I, _I]),
    "nnabla_hip_create_group_normalization": (_P, [_S, _S, _S, _I, _I, _IP, _I, _F, _I, _I]),
    "nnabla_hip_create_instance_normalization": (_P, [_S, _S, _S, _I, _IP, _I, _F, _I, _I]),
    "nnabla_hip_create_tensor_normalization": (_P, [_S, _S, _S, _IP, _I, _F, _I, _I]),
    "nnabla_hip_create_weight_standardization": (_P, [_S, _S, _S, _I, _F]),
    "nnabla_hip_function_delete": (None, [_P]),
    "nnabla_hip_function_name": (_S, [_P]),
    "nnabla_hip_function_setup": (_I, [_P, _PP, _I, _PP, _I]),
    "nnabla_hip_function_forward": (_I, [_P, _PP, _I, _PP, _I]),
    "nnabla_hip_function_recompute": (_I, [_P, _PP, _I, _PP, _I]),
    "nnabla_hip_function_backward": (_I, [_P, _PP, _I, _PP, _I, _IP, _IP]),
}

_lib = None


class NblaError(RuntimeError):
    """An nbla::Exception that crossed the C surface."""

    def __init__(self, code, text):
        super().__init__(text)
        self.code = code


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(HOST_LIB_PATH):
            raise RuntimeError(f"{HOST_LIB_PATH} is missing: build it first (make -C csrc)")
        h = ctypes.CDLL(HOST_LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(h, name)
            fn.restype = res
            fn.argtypes = args
        _lib = h
    return _lib


def _check(code):
    if code != 0:
        raise NblaError(code, lib().nnabla_hip_last_error().decode())


def init():
    _check(lib().nnabla_hip_init())


def set_host_array_class(name):
    """"CpuArray" (default) or "HipCachedHostArray": the host array class
    Variable.d / set_data stage through."""
    _check(lib().nnabla_hip_set_host_array_class(name.encode()))


def array_classes():
    """Array classes of the backend, the default one first
    (python/src/nnabla_ext/cuda/init.pyx:137-138)."""
    init()
    return lib().nnabla_hip_array_classes().decode().split(",")


def context(device_id=0, type_config="float", **kw):
    """Backend preference list the way the reference's context() builds it
    (python/src/nnabla_ext/cuda/__init__.py:138-149): half falls back to
    float.  There is no 'cpu:float' tail: this backend has no CPU path."""
    if type_config == "half":
        backends = ["hip:half", "hip:float"]
    elif type_config == "float":
        backends = ["hip:float"]
    else:
        raise ValueError("Unknown data type config is given %s" % type_config)
    return {"backends": ",".join(backends), "array_class": kw.get("array_class", "HipCachedArray"),
            "device_id": str(device_id)}


ASYNC, UNSAFE = 1, 2


def pending_transfers():
    """Host-to-device transfers whose source array the backend still holds."""
    n = ctypes.c_uint64(0)
    _check(lib().nnabla_hip_pending_transfers(ctypes.byref(n)))
    return n.value


def device_synchronize(device="0"):
    """hipDeviceSynchronize on one device (init.pyx:179-186)."""
    _check(lib().nnabla_hip_device_synchronize(str(device).encode()))


def synchronize(device_id=0, **kw):
    return device_synchronize(device_id)


def get_device_count():
    n = ctypes.c_int(0)
    _check(lib().nnabla_hip_device_count(ctypes.byref(n)))
    return n.value


def get_devices():
    return [str(i) for i in range(get_device_count())]


def clear_memory_cache():
    """Returns every cached device block to the driver (init.pyx:74-75)."""
    _check(lib().nnabla_hip_clear_memory_cache())


def memory_stats():
    """(bytes handed out, bytes held in the cache) of the caching allocator."""
    live, cached = ctypes.c_uint64(0), ctypes.c_uint64(0)
    _check(lib().nnabla_hip_memory_stats(ctypes.byref(live), ctypes.byref(cached)))
    return live.value, cached.value


def _ints(seq):
    arr = (ctypes.c_int * max(len(seq), 1))(*seq)
    return arr, len(seq)


class Variable:
    def __init__(self, shape):
        self.shape = tuple(int(s) for s in shape)
        arr = (_I64 * max(len(self.shape), 1))(*self.shape)
        self._h = lib().nnabla_hip_variable_new(len(self.shape), arr)
        if not self._h:
            raise NblaError(-1, lib().nnabla_hip_last_error().decode())

    def __del__(self):
        # (at interpreter shutdown the module globals may be gone already)
        if getattr(self, "_h", None) and lib is not None:
            lib().nnabla_hip_variable_delete(self._h)
            self._h = None

    @property
    def current_shape(self):
        n = lib().nnabla_hip_variable_ndim(self._h)
        out = (_I64 * max(n, 1))()
        _check(lib().nnabla_hip_variable_shape(self._h, out))
        return tuple(out[i] for i in range(n))

    def _set(self, which, a, half):
        a = np.ascontiguousarray(a, dtype=np.float32).reshape(-1)
        _check(lib().nnabla_hip_variable_set(self._h, which, a.ctypes.data_as(_FP), a.size,
                                             1 if half else 0))

    def _get(self, which):
        shape = self.current_shape
        out = np.empty(int(np.prod(shape, dtype=np.int64)), np.float32)
        _check(lib().nnabla_hip_variable_get(self._h, which, out.ctypes.data_as(_FP), out.size))
        return out.reshape(shape)

    def set_data(self, a, half=False):
        self._set(0, a, half)

    def set_grad(self, a, half=False):
        self._set(1, a, half)

    @property
    def d(self):
        return self._get(0)

    @property
    def g(self):
        return self._get(1)

    def cast(self, array_class, device_id="0", which=0, half=False, write_only=False,
             async_flags=0):
        """NdArray.cast to an array class; async_flags: ASYNC = 1, UNSAFE = 2."""
        _check(lib().nnabla_hip_variable_cast(self._h, which, array_class.encode(),
                                              str(device_id).encode(), 1 if half else 0,
                                              1 if write_only else 0, int(async_flags)))

    # numpy dtype -> 0x100 + the core's dtypes enumerator
    _RAW = {"bool": 0, "int8": 1, "uint8": 2, "int16": 3, "uint16": 4, "int32": 5, "uint32": 6,
            "int64": 7, "uint64": 8, "float32": 9, "float64": 10, "float16": 23}

    def set_raw(self, a, which=0):
        """Stores `a` in its own dtype (no conversion)."""
        a = np.ascontiguousarray(a).reshape(-1)
        _check(lib().nnabla_hip_variable_set_raw(self._h, which, a.ctypes.data, a.size,
                                                 0x100 + self._RAW[a.dtype.name]))

    def get_raw(self, dtype, which=0):
        shape = self.current_shape
        out = np.empty(int(np.prod(shape, dtype=np.int64)), np.dtype(dtype))
        _check(lib().nnabla_hip_variable_get_raw(self._h, which, out.ctypes.data, out.size,
                                                 0x100 + self._RAW[out.dtype.name]))
        return out.reshape(shape)

    def cast_raw(self, array_class, dtype, device_id="0", which=0, async_flags=0):
        _check(lib().nnabla_hip_variable_cast(self._h, which, array_class.encode(),
                                              str(device_id).encode(),
                                              0x100 + self._RAW[np.dtype(dtype).name], 0,
                                              int(async_flags)))

    def zero_data(self):
        _check(lib().nnabla_hip_variable_zero(self._h, 0))

    def zero_grad(self):
        _check(lib().nnabla_hip_variable_zero(self._h, 1))

    def stored_dtype(self, which=0):
        """"float", "half", "other" or None (nothing stored yet) of data (0) / grad (1)."""
        d = _I(0)
        _check(lib().nnabla_hip_variable_stored_dtype(self._h, which, ctypes.byref(d)))
        return {0: "float", 1: "half", -1: None}.get(d.value, "other")

    def fill_grad(self, v):
        _check(lib().nnabla_hip_variable_fill(self._h, 1, float(v)))

    def fill_data(self, v):
        _check(lib().nnabla_hip_variable_fill(self._h, 0, float(v)))


def _handles(vs):
    arr = (ctypes.c_void_p * max(len(vs), 1))(*[v._h for v in vs])
    return ctypes.cast(arr, _PP), len(vs)


class Function:
    def __init__(self, handle):
        if not handle:
            raise NblaError(-1, lib().nnabla_hip_last_error().decode())
        self._h = handle

    def __del__(self):
        if getattr(self, "_h", None) and lib is not None:
            lib().nnabla_hip_function_delete(self._h)
            self._h = None

    @property
    def name(self):
        return lib().nnabla_hip_function_name(self._h).decode()

    def setup(self, inputs, outputs):
        i, ni = _handles(inputs)
        o, no = _handles(outputs)
        _check(lib().nnabla_hip_function_setup(self._h, i, ni, o, no))

    def forward(self, inputs, outputs):
        i, ni = _handles(inputs)
        o, no = _handles(outputs)
        _check(lib().nnabla_hip_function_forward(self._h, i, ni, o, no))

    def recompute(self, inputs, outputs):
        i, ni = _handles(inputs)
        o, no = _handles(outputs)
        _check(lib().nnabla_hip_function_recompute(self._h, i, ni, o, no))

    def backward(self, inputs, outputs, propagate_down=None, accum=None):
        i, ni = _handles(inputs)
        o, no = _handles(outputs)
        pd = [1] * ni if propagate_down is None else [int(bool(p)) for p in propagate_down]
        ac = [0] * ni if accum is None else [int(bool(a)) for a in accum]
        pda, _ = _ints(pd)
        aca, _ = _ints(ac)
        _check(lib().nnabla_hip_function_backward(self._h, i, ni, o, no, pda, aca))


def _ctx_args(ctx):
    return ctx["backends"].encode(), ctx["array_class"].encode(), ctx["device_id"].encode()


def BatchNormalization(ctx, axes=(1,), decay_rate=0.9, eps=1e-5, batch_stat=True, no_scale=False,
                       no_bias=False):
    ax, n = _ints(list(axes))
    return Function(lib().nnabla_hip_create_batch_normalization(
        *_ctx_args(ctx), ax, n, decay_rate, eps, int(batch_stat), int(no_scale), int(no_bias)))


def FusedBatchNormalization(ctx, axes=(1,), decay_rate=0.9, eps=1e-5, batch_stat=True,
                            nonlinearity="relu"):
    ax, n = _ints(list(axes))
    return Function(lib().nnabla_hip_create_fused_batch_normalization(
        *_ctx_args(ctx), ax, n, decay_rate, eps, int(batch_stat), nonlinearity.encode()))


def LayerNormalization(ctx, batch_axis=(0,), eps=1e-5, no_scale=False, no_bias=False):
    ba, n = _ints(list(batch_axis))
    return Function(lib().nnabla_hip_create_layer_normalization(
        *_ctx_args(ctx), ba, n, eps, int(no_scale), int(no_bias)))


def GroupNormalization(ctx, num_groups=1, channel_axis=1, batch_axis=(0,), eps=1e-5, no_scale=False,
                       no_bias=False):
    ba, n = _ints(list(batch_axis))
    return Function(lib().nnabla_hip_create_group_normalization(
        *_ctx_args(ctx), num_groups, channel_axis, ba, n, eps, int(no_scale), int(no_bias)))


def InstanceNormalization(ctx, channel_axis=1, batch_axis=(0,), eps=1e-5, no_scale=False,
                          no_bias=False):
    ba, n = _ints(list(batch_axis))
    return Function(lib().nnabla_hip_create_instance_normalization(
        *_ctx_args(ctx), channel_axis, ba, n, eps, int(no_scale), int(no_bias)))


def TensorNormalization(ctx, axes=(1,), eps=1e-5, no_scale=False, no_bias=False):
    """axes: the axes the statistics keep (adjacent); beta/gamma have their extent."""
    ax, n = _ints(list(axes))
    return Function(lib().nnabla_hip_create_tensor_normalization(
        *_ctx_args(ctx), ax, n, eps, int(no_scale), int(no_bias)))


def WeightStandardization(ctx, channel_axis=0, eps=1e-5):
    return Function(lib().nnabla_hip_create_weight_standardization(
        *_ctx_args(ctx), channel_axis, eps))
