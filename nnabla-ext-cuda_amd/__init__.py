"""ctypes binding of the nblahip C-ABI (include/nblahip.h) for tests, the
smoke check and the benchmark.

The product is the C/C++ library; this module only hands it device pointers.
torch supplies device memory and the current stream, nothing else: there is
no fallback implementation here, and loading fails loudly when the HIP
library has not been built.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libnblahip.so")
HOST_LIB_PATH = os.path.join(_HERE, "lib", "libnnabla_hip.so")
CSRC = os.path.join(_HERE, "csrc")

F32, F16 = 0, 1

_c_void_p = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_f = ctypes.c_float
_sz = ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/nblahip.h one to one.
SIGNATURES = {
    "nblahip_error_string": (ctypes.c_char_p, [_int]),
    "nblahip_abi_version": (_int, []),
    "nblahip_bn_fwd_infer": (_int, [_c_void_p] * 6 + [_i64] * 3 + [_f, _int, _c_void_p]),
    "nblahip_bn_workspace_bytes": (_sz, [_i64] * 3 + [_int]),
    "nblahip_bn_fwd_train": (_int, [_c_void_p] * 8 + [_i64] * 3 + [_f, _f, _int, _c_void_p, _sz,
                                                              _c_void_p]),
    "nblahip_bn_fwd_train_static_max_workspace": (_sz, []),
    "nblahip_bn_fwd_train_static": (_int, [_c_void_p] * 8 + [_i64] * 3 + [_f, _f, _int, _c_void_p]),
    "nblahip_bn_bwd": (_int, [_c_void_p] * 10 + [_int] * 3 + [_i64] * 3 + [_f, _int, _int,
                                                                   _c_void_p, _sz, _c_void_p]),
    "nblahip_bn_local_stats": (_int, [_c_void_p] * 3 + [_i64] * 3 + [_int, _c_void_p, _sz, _c_void_p]),
    "nblahip_bn_merge_stats": (_int, [_c_void_p, _int, _i64] + [_c_void_p] * 4 + [_f, _c_void_p]),
    "nblahip_bn_bwd_local_sums": (_int, [_c_void_p] * 7 + [_int, _int] + [_i64] * 3 + [_f, _int,
                                                                          _c_void_p, _sz, _c_void_p]),
    "nblahip_bn_bwd_apply_sums": (_int, [_c_void_p] * 6 + [ctypes.c_double] + [_c_void_p] * 3 +
                                  [_int] + [_i64] * 3 + [_f, _int, _c_void_p, _sz, _c_void_p]),
    "nblahip_fused_bn_fwd_infer": (_int, [_c_void_p] * 7 + [_i64] * 3 + [_f, _int, _c_void_p]),
    "nblahip_fused_bn_fwd_train": (_int, [_c_void_p] * 9 + [_i64] * 3 + [_f, _f, _int, _c_void_p,
                                                                         _sz, _c_void_p]),
    "nblahip_fused_bn_bwd": (_int, [_c_void_p] * 12 + [_int] * 4 + [_i64] * 3 + [_f, _int, _int,
                                                                         _c_void_p, _sz, _c_void_p]),
    "nblahip_ln_fwd": (_int, [_c_void_p] * 6 + [_i64] * 2 + [_f, _int, _c_void_p]),
    "nblahip_ln_bwd_workspace_bytes": (_sz, [_i64] * 2 + [_int]),
    "nblahip_ln_bwd": (_int, [_c_void_p] * 10 + [_int] * 3 + [_i64] * 2 + [_f, _int, _c_void_p,
                                                                   _sz, _c_void_p]),
    "nblahip_gn_fwd": (_int, [_c_void_p] * 6 + [_i64] * 3 + [_int, _f, _int, _c_void_p]),
    "nblahip_gn_bwd_workspace_bytes": (_sz, [_i64] * 3 + [_int, _int]),
    "nblahip_gn_bwd": (_int, [_c_void_p] * 10 + [_int] * 3 + [_i64] * 3 + [_int, _f, _int,
                                                                   _c_void_p, _sz, _c_void_p]),
    "nblahip_in_fwd": (_int, [_c_void_p] * 6 + [_i64] * 3 + [_int, _int, _f, _int, _c_void_p]),
    "nblahip_in_bwd_workspace_bytes": (_sz, [_i64] * 3 + [_int]),
    "nblahip_in_bwd": (_int, [_c_void_p] * 10 + [_int] * 3 + [_i64] * 3 + [_int, _int, _f, _int,
                                                                   _c_void_p, _sz, _c_void_p]),
    "nblahip_gn_cl_workspace_bytes": (_sz, [_i64] * 3 + [_int, _int]),
    "nblahip_gn_cl_fwd": (_int, [_c_void_p] * 6 + [_i64] * 3 + [_int, _f, _int, _c_void_p, _sz,
                                                                _c_void_p]),
    "nblahip_gn_cl_bwd": (_int, [_c_void_p] * 10 + [_int] * 3 + [_i64] * 3 + [_int, _f, _int,
                                                                      _c_void_p, _sz, _c_void_p]),
    "nblahip_in_cl_workspace_bytes": (_sz, [_i64] * 3 + [_int]),
    "nblahip_in_cl_fwd": (_int, [_c_void_p] * 6 + [_i64] * 3 + [_int, _int, _f, _int, _c_void_p,
                                                                _sz, _c_void_p]),
    "nblahip_in_cl_bwd": (_int, [_c_void_p] * 10 + [_int] * 3 + [_i64] * 3 + [_int, _int, _f, _int,
                                                                      _c_void_p, _sz, _c_void_p]),
    "nblahip_device_count": (_int, [ctypes.POINTER(_int)]),
    "nblahip_set_device": (_int, [_int]),
    "nblahip_get_device": (_int, [ctypes.POINTER(_int)]),
    "nblahip_device_synchronize": (_int, []),
    "nblahip_stream_synchronize": (_int, [_c_void_p]),
    "nblahip_device_info": (_int, [_int, ctypes.c_char_p, _sz, ctypes.POINTER(_int),
                                   ctypes.POINTER(_int), ctypes.POINTER(_sz)]),
    "nblahip_malloc": (_int, [ctypes.POINTER(_c_void_p), _sz]),
    "nblahip_free": (_int, [_c_void_p]),
    "nblahip_host_malloc": (_int, [ctypes.POINTER(_c_void_p), _sz]),
    "nblahip_host_free": (_int, [_c_void_p]),
    "nblahip_memcpy_h2d": (_int, [_c_void_p, _c_void_p, _sz, _c_void_p]),
    "nblahip_memcpy_d2h": (_int, [_c_void_p, _c_void_p, _sz, _c_void_p]),
    "nblahip_memcpy_d2d": (_int, [_c_void_p, _c_void_p, _sz, _c_void_p]),
    "nblahip_memcpy_h2d_async": (_int, [_c_void_p, _c_void_p, _sz, _c_void_p]),
    "nblahip_memcpy_d2h_async": (_int, [_c_void_p, _c_void_p, _sz, _c_void_p]),
    "nblahip_stream_create": (_int, [ctypes.POINTER(_c_void_p)]),
    "nblahip_stream_destroy": (_int, [_c_void_p]),
    "nblahip_event_create": (_int, [ctypes.POINTER(_c_void_p)]),
    "nblahip_event_destroy": (_int, [_c_void_p]),
    "nblahip_event_record": (_int, [_c_void_p, _c_void_p]),
    "nblahip_stream_wait_event": (_int, [_c_void_p, _c_void_p]),
    "nblahip_event_synchronize": (_int, [_c_void_p]),
    "nblahip_event_query": (_int, [_c_void_p, ctypes.POINTER(_int)]),
    "nblahip_memset": (_int, [_c_void_p, _int, _sz, _c_void_p]),
    "nblahip_convert": (_int, [_c_void_p, _int, _c_void_p, _int, _i64, _c_void_p]),
    "nblahip_fill": (_int, [_c_void_p, _int, _f, _i64, _c_void_p]),
    "nblahip_fill_bytes": (_int, [_c_void_p, _int, ctypes.c_ulonglong, _i64, _c_void_p]),
    "nblahip_permute": (_int, [_c_void_p, _c_void_p, _int, ctypes.POINTER(_i64),
                               ctypes.POINTER(_int), _int, _int, _c_void_p]),
    "nblahip_profile_enable": (_int, [_int]),
    "nblahip_profile_reset": (_int, []),
    "nblahip_profile_query": (_int, [ctypes.c_char_p, ctypes.POINTER(ctypes.c_double),
                                     ctypes.POINTER(_i64)]),
    "nblahip_profile_kernels": (_int, [ctypes.c_char_p, _sz, ctypes.POINTER(_sz)]),
    "nblahip_tune_set": (_int, [ctypes.c_char_p, _int]),
    "nblahip_tune_get": (_int, [ctypes.c_char_p, _int]),
    "nblahip_tune_reset": (_int, []),
    "nblahip_xchg_set_epoch": (_int, [ctypes.c_uint]),
    "nblahip_stage_params": (_int, [_int, ctypes.POINTER(_c_void_p), _int, ctypes.POINTER(_c_void_p),
                                    _int, ctypes.POINTER(_i64), _c_void_p]),
}

_lib = None


class NblaHipError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"nblahip status {code}: {text}")
        self.code = code


def lib():
    """The loaded libnblahip.so.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {CSRC} -j8` "
                "(or __graft_entry__.build()); there is no fallback path")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(code):
    if code != 0:
        raise NblaHipError(code, lib().nblahip_error_string(code).decode())


def profile_query(kernel_name):
    """(total_ms, launches) of the recorded launches of one kernel."""
    total = ctypes.c_double(0.0)
    count = _i64(0)
    check(lib().nblahip_profile_query(kernel_name.encode(), ctypes.byref(total),
                                      ctypes.byref(count)))
    return total.value, count.value


def profile_kernels():
    """Names of the kernels recorded since the last profile reset, in order of
    first launch."""
    need = _sz(0)
    check(lib().nblahip_profile_kernels(None, 0, ctypes.byref(need)))
    buf = ctypes.create_string_buffer(need.value)
    check(lib().nblahip_profile_kernels(buf, need.value, ctypes.byref(need)))
    return [n for n in buf.value.decode().split("\n") if n]


def tune_set(name, value):
    """Override plan knob NBLAHIP_<name> from the next call on (-1: undo)."""
    check(lib().nblahip_tune_set(name.encode(), int(value)))


def tune_get(name, fallback=-1):
    return lib().nblahip_tune_get(name.encode(), int(fallback))


def tune_reset():
    check(lib().nblahip_tune_reset())


# ---------------------------------------------------------------------------
# torch-tensor conveniences (device memory + current stream only)
# ---------------------------------------------------------------------------
def _ptr(t):
    return None if t is None else t.data_ptr()


def _stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def _dtype_code(t):
    import torch
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.float16:
        return F16
    raise TypeError(f"unsupported activation dtype {t.dtype}")


def _f32(t, name):
    import torch
    if t is not None and (t.dtype != torch.float32 or not t.is_contiguous()):
        raise TypeError(f"{name} must be a contiguous float32 tensor")
    return t


def _workspace(nbytes, device):
    import torch
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


def _bn_sizes(shape, axis):
    size0 = 1
    for s in shape[:axis]:
        size0 *= s
    size2 = 1
    for s in shape[axis + 1:]:
        size2 *= s
    return size0, shape[axis], size2


def bn_forward_global(x, beta, gamma, rmean, rvar, axis=1, eps=1e-5):
    import torch
    assert x.is_contiguous()
    s0, c, s2 = _bn_sizes(x.shape, axis)
    y = torch.empty_like(x)
    check(lib().nblahip_bn_fwd_infer(_ptr(x), _ptr(_f32(rmean, "rmean")), _ptr(_f32(rvar, "rvar")),
                                     _ptr(_f32(gamma, "gamma")), _ptr(_f32(beta, "beta")), _ptr(y),
                                     s0, c, s2, eps, _dtype_code(x), _stream()))
    return y


def bn_forward_batch(x, beta, gamma, rmean, rvar, axis=1, decay_rate=0.9, eps=1e-5, ws=None,
                     y=None):
    """Returns y, batch_mean, batch_var; rmean/rvar are updated in place.
    y: the output tensor (x itself for an in-place call); allocated when None."""
    import torch
    assert x.is_contiguous()
    s0, c, s2 = _bn_sizes(x.shape, axis)
    dt = _dtype_code(x)
    y = torch.empty_like(x) if y is None else y
    mean = torch.empty(c, dtype=torch.float32, device=x.device)
    var = torch.empty(c, dtype=torch.float32, device=x.device)
    need = lib().nblahip_bn_workspace_bytes(s0, c, s2, dt)
    ws = ws if ws is not None else _workspace(need, x.device)
    check(lib().nblahip_bn_fwd_train(_ptr(x), _ptr(_f32(gamma, "gamma")), _ptr(_f32(beta, "beta")),
                                     _ptr(y), _ptr(mean), _ptr(var), _ptr(_f32(rmean, "rmean")),
                                     _ptr(_f32(rvar, "rvar")), s0, c, s2, decay_rate, eps, dt,
                                     _ptr(ws), ws.numel(), _stream()))
    return y, mean, var


def bn_forward_batch_static(x, beta, gamma, rmean, rvar, axis=1, decay_rate=0.9, eps=1e-5,
                            out=None):
    """bn_forward_batch through the entry point that allocates nothing; out =
    (y, mean, var) preallocated by the caller (allocated here when None)."""
    import torch
    assert x.is_contiguous()
    s0, c, s2 = _bn_sizes(x.shape, axis)
    if out is None:
        out = (torch.empty_like(x), torch.empty(c, dtype=torch.float32, device=x.device),
               torch.empty(c, dtype=torch.float32, device=x.device))
    y, mean, var = out
    check(lib().nblahip_bn_fwd_train_static(
        _ptr(x), _ptr(_f32(gamma, "gamma")), _ptr(_f32(beta, "beta")), _ptr(y), _ptr(mean),
        _ptr(var), _ptr(_f32(rmean, "rmean")), _ptr(_f32(rvar, "rvar")), s0, c, s2, decay_rate,
        eps, _dtype_code(x), _stream()))
    return y, mean, var


def bn_backward(x, dy, gamma, mean, var, axis=1, eps=1e-5, batch_stat=True, dmean=None,
                dvar=None, dx=None, dgamma=None, dbeta=None, accum=(False, False, False),
                need=(True, True, True), ws=None):
    """need = (dx, dgamma, dbeta) propagate_down flags; accum likewise.
    Returns dx, dgamma, dbeta (None where not needed)."""
    import torch
    assert x.is_contiguous() and dy.is_contiguous()
    s0, c, s2 = _bn_sizes(x.shape, axis)
    dt = _dtype_code(x)
    if need[0] and dx is None:
        dx = torch.empty_like(x)
    if need[1] and dgamma is None:
        dgamma = torch.empty(c, dtype=torch.float32, device=x.device)
    if need[2] and dbeta is None:
        dbeta = torch.empty(c, dtype=torch.float32, device=x.device)
    nbytes = lib().nblahip_bn_workspace_bytes(s0, c, s2, dt)
    ws = ws if ws is not None else _workspace(nbytes, x.device)
    check(lib().nblahip_bn_bwd(_ptr(x), _ptr(dy), _ptr(_f32(gamma, "gamma")), _ptr(mean), _ptr(var),
                               _ptr(dmean), _ptr(dvar), _ptr(dx if need[0] else None),
                               _ptr(dgamma if need[1] else None), _ptr(dbeta if need[2] else None),
                               int(accum[0]), int(accum[1]), int(accum[2]), s0, c, s2, eps,
                               int(batch_stat), dt, _ptr(ws), ws.numel(), _stream()))
    return (dx if need[0] else None, dgamma if need[1] else None, dbeta if need[2] else None)


def bn_local_stats(x, axis=1, ws=None):
    """mean[C], biased var[C] of this shard of the batch."""
    import torch
    assert x.is_contiguous()
    s0, c, s2 = _bn_sizes(x.shape, axis)
    dt = _dtype_code(x)
    mean = torch.empty(c, dtype=torch.float32, device=x.device)
    var = torch.empty(c, dtype=torch.float32, device=x.device)
    need = lib().nblahip_bn_workspace_bytes(s0, c, s2, dt)
    ws = ws if ws is not None else _workspace(need, x.device)
    check(lib().nblahip_bn_local_stats(_ptr(x), _ptr(mean), _ptr(var), s0, c, s2, dt, _ptr(ws),
                                       ws.numel(), _stream()))
    return mean, var


def bn_merge_stats(stats, channels, rmean=None, rvar=None, decay_rate=0.9):
    """stats: float32 [workers, 2*channels+1] = {mean, var, count} per worker."""
    import torch
    assert stats.is_contiguous() and stats.dtype == torch.float32
    mean = torch.empty(channels, dtype=torch.float32, device=stats.device)
    var = torch.empty(channels, dtype=torch.float32, device=stats.device)
    check(lib().nblahip_bn_merge_stats(_ptr(stats), stats.shape[0], channels, _ptr(mean), _ptr(var),
                                       _ptr(_f32(rmean, "rmean")), _ptr(_f32(rvar, "rvar")),
                                       decay_rate, _stream()))
    return mean, var


def bn_backward_local_sums(x, dy, mean, var, axis=1, eps=1e-5, need_params=True, ws=None):
    """Returns sums[C, 2] = (sum dy*(x-mean), sum dy) of this shard, dgamma, dbeta."""
    import torch
    assert x.is_contiguous() and dy.is_contiguous()
    s0, c, s2 = _bn_sizes(x.shape, axis)
    dt = _dtype_code(x)
    sums = torch.empty(c, 2, dtype=torch.float32, device=x.device)
    dg = torch.empty(c, dtype=torch.float32, device=x.device) if need_params else None
    db = torch.empty(c, dtype=torch.float32, device=x.device) if need_params else None
    need = lib().nblahip_bn_workspace_bytes(s0, c, s2, dt)
    ws = ws if ws is not None else _workspace(need, x.device)
    check(lib().nblahip_bn_bwd_local_sums(_ptr(x), _ptr(dy), _ptr(mean), _ptr(var), _ptr(sums),
                                          _ptr(dg), _ptr(db), 0, 0, s0, c, s2, eps, dt, _ptr(ws),
                                          ws.numel(), _stream()))
    return sums, dg, db


def bn_backward_apply_sums(x, dy, gamma, mean, var, sums, total_count, axis=1, eps=1e-5,
                           dmean=None, dvar=None, dx=None, accum=False, ws=None):
    import torch
    assert x.is_contiguous() and dy.is_contiguous() and sums.is_contiguous()
    s0, c, s2 = _bn_sizes(x.shape, axis)
    dt = _dtype_code(x)
    if dx is None:
        dx = torch.empty_like(x)
    need = lib().nblahip_bn_workspace_bytes(s0, c, s2, dt)
    ws = ws if ws is not None else _workspace(need, x.device)
    check(lib().nblahip_bn_bwd_apply_sums(_ptr(x), _ptr(dy), _ptr(_f32(gamma, "gamma")), _ptr(mean),
                                          _ptr(var), _ptr(sums), float(total_count), _ptr(dmean),
                                          _ptr(dvar), _ptr(dx), int(accum), s0, c, s2, eps, dt,
                                          _ptr(ws), ws.numel(), _stream()))
    return dx


def fused_bn_forward_global(x, z, beta, gamma, rmean, rvar, axis=1, eps=1e-5):
    """y = max(0, bn_inference(x) + z); z may be None."""
    import torch
    assert x.is_contiguous() and (z is None or z.is_contiguous())
    s0, c, s2 = _bn_sizes(x.shape, axis)
    y = torch.empty_like(x)
    check(lib().nblahip_fused_bn_fwd_infer(
        _ptr(x), _ptr(z), _ptr(_f32(rmean, "rmean")), _ptr(_f32(rvar, "rvar")),
        _ptr(_f32(gamma, "gamma")), _ptr(_f32(beta, "beta")), _ptr(y), s0, c, s2, eps,
        _dtype_code(x), _stream()))
    return y


def fused_bn_forward_batch(x, z, beta, gamma, rmean, rvar, axis=1, decay_rate=0.9, eps=1e-5,
                           ws=None):
    """y = max(0, bn_training(x) + z); returns y, batch_mean, batch_var."""
    import torch
    assert x.is_contiguous() and (z is None or z.is_contiguous())
    s0, c, s2 = _bn_sizes(x.shape, axis)
    dt = _dtype_code(x)
    y = torch.empty_like(x)
    mean = torch.empty(c, dtype=torch.float32, device=x.device)
    var = torch.empty(c, dtype=torch.float32, device=x.device)
    need = lib().nblahip_bn_workspace_bytes(s0, c, s2, dt)
    ws = ws if ws is not None else _workspace(need, x.device)
    check(lib().nblahip_fused_bn_fwd_train(
        _ptr(x), _ptr(z), _ptr(_f32(gamma, "gamma")), _ptr(_f32(beta, "beta")), _ptr(y),
        _ptr(mean), _ptr(var), _ptr(_f32(rmean, "rmean")), _ptr(_f32(rvar, "rvar")), s0, c, s2,
        decay_rate, eps, dt, _ptr(ws), ws.numel(), _stream()))
    return y, mean, var


def fused_bn_backward(x, y, dy, gamma, mean, var, axis=1, eps=1e-5, batch_stat=True, dmean=None,
                      dvar=None, dx=None, dz=None, dgamma=None, dbeta=None,
                      accum=(False, False, False, False), need=(True, True, True, True), ws=None):
    """need / accum = (dx, dz, dgamma, dbeta).  Returns dx, dz, dgamma, dbeta."""
    import torch
    assert x.is_contiguous() and dy.is_contiguous() and y.is_contiguous()
    s0, c, s2 = _bn_sizes(x.shape, axis)
    dt = _dtype_code(x)
    if need[0] and dx is None:
        dx = torch.empty_like(x)
    if need[1] and dz is None:
        dz = torch.empty_like(x)
    if need[2] and dgamma is None:
        dgamma = torch.empty(c, dtype=torch.float32, device=x.device)
    if need[3] and dbeta is None:
        dbeta = torch.empty(c, dtype=torch.float32, device=x.device)
    nbytes = lib().nblahip_bn_workspace_bytes(s0, c, s2, dt)
    ws = ws if ws is not None else _workspace(nbytes, x.device)
    check(lib().nblahip_fused_bn_bwd(
        _ptr(x), _ptr(y), _ptr(dy), _ptr(_f32(gamma, "gamma")), _ptr(mean), _ptr(var), _ptr(dmean),
        _ptr(dvar), _ptr(dx if need[0] else None), _ptr(dz if need[1] else None),
        _ptr(dgamma if need[2] else None), _ptr(dbeta if need[3] else None), int(accum[0]),
        int(accum[1]), int(accum[2]), int(accum[3]), s0, c, s2, eps, int(batch_stat), dt, _ptr(ws),
        ws.numel(), _stream()))
    return (dx if need[0] else None, dz if need[1] else None, dgamma if need[2] else None,
            dbeta if need[3] else None)


def ln_forward(x, beta, gamma, outer, eps=1e-5):
    import torch
    assert x.is_contiguous()
    reduce = x.numel() // outer if outer else 0
    y = torch.empty_like(x)
    mean = torch.empty(outer, dtype=torch.float32, device=x.device)
    var = torch.empty(outer, dtype=torch.float32, device=x.device)
    check(lib().nblahip_ln_fwd(_ptr(x), _ptr(_f32(gamma, "gamma")), _ptr(_f32(beta, "beta")),
                               _ptr(y), _ptr(mean), _ptr(var), outer, reduce, eps, _dtype_code(x),
                               _stream()))
    return y, mean, var


def ln_backward(x, dy, gamma, mean, var, outer, eps=1e-5, dmean=None, dvar=None, dx=None,
                dgamma=None, dbeta=None, accum=(False, False, False), need=(True, True, True),
                ws=None):
    import torch
    assert x.is_contiguous() and dy.is_contiguous()
    reduce = x.numel() // outer if outer else 0
    dt = _dtype_code(x)
    if need[0] and dx is None:
        dx = torch.empty_like(x)
    if need[1] and dgamma is None:
        dgamma = torch.empty(reduce, dtype=torch.float32, device=x.device)
    if need[2] and dbeta is None:
        dbeta = torch.empty(reduce, dtype=torch.float32, device=x.device)
    nbytes = lib().nblahip_ln_bwd_workspace_bytes(outer, reduce, dt)
    ws = ws if ws is not None else _workspace(nbytes, x.device)
    check(lib().nblahip_ln_bwd(_ptr(x), _ptr(dy), _ptr(_f32(gamma, "gamma")), _ptr(mean), _ptr(var),
                               _ptr(dmean), _ptr(dvar), _ptr(dx if need[0] else None),
                               _ptr(dgamma if need[1] else None), _ptr(dbeta if need[2] else None),
                               int(accum[0]), int(accum[1]), int(accum[2]), outer, reduce, eps, dt,
                               _ptr(ws), ws.numel(), _stream()))
    return (dx if need[0] else None, dgamma if need[1] else None, dbeta if need[2] else None)


def _ncs(x, channel_last=False):
    """(batch, channels, spatial) of [N, C, *spatial] or, channel-last, [N, *spatial, C]."""
    n = x.shape[0]
    c = x.shape[-1] if channel_last else x.shape[1]
    sp = 1
    for s in (x.shape[1:-1] if channel_last else x.shape[2:]):
        sp *= s
    return n, c, sp


def gn_forward(x, beta, gamma, num_groups, eps=1e-5, channel_last=False, ws=None, y=None):
    import torch
    assert x.is_contiguous()
    n, c, sp = _ncs(x, channel_last)
    y = torch.empty_like(x) if y is None else y
    mean = torch.empty(n * num_groups, dtype=torch.float32, device=x.device)
    var = torch.empty(n * num_groups, dtype=torch.float32, device=x.device)
    if channel_last:
        dt = _dtype_code(x)
        nbytes = lib().nblahip_gn_cl_workspace_bytes(n, sp, c, num_groups, dt)
        ws = ws if ws is not None else _workspace(nbytes, x.device)
        check(lib().nblahip_gn_cl_fwd(_ptr(x), _ptr(_f32(gamma, "gamma")),
                                      _ptr(_f32(beta, "beta")), _ptr(y), _ptr(mean), _ptr(var),
                                      n, sp, c, num_groups, eps, dt, _ptr(ws), ws.numel(),
                                      _stream()))
        return y, mean, var
    check(lib().nblahip_gn_fwd(_ptr(x), _ptr(_f32(gamma, "gamma")), _ptr(_f32(beta, "beta")),
                               _ptr(y), _ptr(mean), _ptr(var), n, c, sp, num_groups, eps,
                               _dtype_code(x), _stream()))
    return y, mean, var


def gn_backward(x, dy, gamma, mean, var, num_groups, eps=1e-5, dmean=None, dvar=None, dx=None,
                dgamma=None, dbeta=None, accum=(False, False, False), need=(True, True, True),
                ws=None, channel_last=False):
    import torch
    assert x.is_contiguous() and dy.is_contiguous()
    n, c, sp = _ncs(x, channel_last)
    dt = _dtype_code(x)
    if need[0] and dx is None:
        dx = torch.empty_like(x)
    if need[1] and dgamma is None:
        dgamma = torch.empty(c, dtype=torch.float32, device=x.device)
    if need[2] and dbeta is None:
        dbeta = torch.empty(c, dtype=torch.float32, device=x.device)
    if channel_last:
        nbytes = lib().nblahip_gn_cl_workspace_bytes(n, sp, c, num_groups, dt)
        ws = ws if ws is not None else _workspace(nbytes, x.device)
        check(lib().nblahip_gn_cl_bwd(
            _ptr(x), _ptr(dy), _ptr(_f32(gamma, "gamma")), _ptr(mean), _ptr(var), _ptr(dmean),
            _ptr(dvar), _ptr(dx if need[0] else None), _ptr(dgamma if need[1] else None),
            _ptr(dbeta if need[2] else None), int(accum[0]), int(accum[1]), int(accum[2]), n, sp, c,
            num_groups, eps, dt, _ptr(ws), ws.numel(), _stream()))
        return (dx if need[0] else None, dgamma if need[1] else None, dbeta if need[2] else None)
    nbytes = lib().nblahip_gn_bwd_workspace_bytes(n, c, sp, num_groups, dt)
    ws = ws if ws is not None else _workspace(nbytes, x.device)
    check(lib().nblahip_gn_bwd(_ptr(x), _ptr(dy), _ptr(_f32(gamma, "gamma")), _ptr(mean), _ptr(var),
                               _ptr(dmean), _ptr(dvar), _ptr(dx if need[0] else None),
                               _ptr(dgamma if need[1] else None), _ptr(dbeta if need[2] else None),
                               int(accum[0]), int(accum[1]), int(accum[2]), n, c, sp, num_groups,
                               eps, dt, _ptr(ws), ws.numel(), _stream()))
    return (dx if need[0] else None, dgamma if need[1] else None, dbeta if need[2] else None)


def in_forward(x, beta, gamma, eps=1e-5, bc_gamma=True, bc_beta=True, channel_last=False,
               ws=None, y=None):
    import torch
    assert x.is_contiguous()
    n, c, sp = _ncs(x, channel_last)
    y = torch.empty_like(x) if y is None else y
    mean = torch.empty(n * c, dtype=torch.float32, device=x.device)
    var = torch.empty(n * c, dtype=torch.float32, device=x.device)
    if channel_last:
        dt = _dtype_code(x)
        nbytes = lib().nblahip_in_cl_workspace_bytes(n, sp, c, dt)
        ws = ws if ws is not None else _workspace(nbytes, x.device)
        check(lib().nblahip_in_cl_fwd(_ptr(x), _ptr(_f32(gamma, "gamma")),
                                      _ptr(_f32(beta, "beta")), _ptr(y), _ptr(mean), _ptr(var),
                                      n, sp, c, int(bc_gamma), int(bc_beta), eps, dt, _ptr(ws),
                                      ws.numel(), _stream()))
        return y, mean, var
    check(lib().nblahip_in_fwd(_ptr(x), _ptr(_f32(gamma, "gamma")), _ptr(_f32(beta, "beta")),
                               _ptr(y), _ptr(mean), _ptr(var), n, c, sp, int(bc_gamma),
                               int(bc_beta), eps, _dtype_code(x), _stream()))
    return y, mean, var


def in_backward(x, dy, gamma, mean, var, eps=1e-5, bc_gamma=True, bc_beta=True, dmean=None,
                dvar=None, dx=None, dgamma=None, dbeta=None, accum=(False, False, False),
                need=(True, True, True), ws=None, channel_last=False):
    import torch
    assert x.is_contiguous() and dy.is_contiguous()
    n, c, sp = _ncs(x, channel_last)
    dt = _dtype_code(x)
    if need[0] and dx is None:
        dx = torch.empty_like(x)
    if need[1] and dgamma is None:
        dgamma = torch.empty(c if bc_gamma else n * c, dtype=torch.float32, device=x.device)
    if need[2] and dbeta is None:
        dbeta = torch.empty(c if bc_beta else n * c, dtype=torch.float32, device=x.device)
    if channel_last:
        nbytes = lib().nblahip_in_cl_workspace_bytes(n, sp, c, dt)
        ws = ws if ws is not None else _workspace(nbytes, x.device)
        check(lib().nblahip_in_cl_bwd(
            _ptr(x), _ptr(dy), _ptr(_f32(gamma, "gamma")), _ptr(mean), _ptr(var), _ptr(dmean),
            _ptr(dvar), _ptr(dx if need[0] else None), _ptr(dgamma if need[1] else None),
            _ptr(dbeta if need[2] else None), int(accum[0]), int(accum[1]), int(accum[2]), n, sp, c,
            int(bc_gamma), int(bc_beta), eps, dt, _ptr(ws), ws.numel(), _stream()))
        return (dx if need[0] else None, dgamma if need[1] else None, dbeta if need[2] else None)
    nbytes = lib().nblahip_in_bwd_workspace_bytes(n, c, sp, dt)
    ws = ws if ws is not None else _workspace(nbytes, x.device)
    check(lib().nblahip_in_bwd(_ptr(x), _ptr(dy), _ptr(_f32(gamma, "gamma")), _ptr(mean), _ptr(var),
                               _ptr(dmean), _ptr(dvar), _ptr(dx if need[0] else None),
                               _ptr(dgamma if need[1] else None), _ptr(dbeta if need[2] else None),
                               int(accum[0]), int(accum[1]), int(accum[2]), n, c, sp,
                               int(bc_gamma), int(bc_beta), eps, dt, _ptr(ws), ws.numel(),
                               _stream()))
    return (dx if need[0] else None, dgamma if need[1] else None, dbeta if need[2] else None)


def permute(x, perm, out=None, accum=False):
    """out (+)= x.permute(perm), contiguous (nblahip_permute)."""
    import torch
    assert x.is_contiguous()
    nd = x.dim()
    shape = (_i64 * nd)(*x.shape)
    pm = (_int * nd)(*perm)
    if out is None:
        out = torch.empty([x.shape[p] for p in perm], dtype=x.dtype, device=x.device)
    check(lib().nblahip_permute(_ptr(x), _ptr(out), nd, shape, pm, int(accum), _dtype_code(x),
                                _stream()))
    return out
