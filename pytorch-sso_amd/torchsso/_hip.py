"""ctypes binding of libkfac_hip.so, the hand-written HIP (gfx950) K-FAC engine.

There is no fallback: if the library is missing, or a tensor is not a
contiguous fp32 tensor on a HIP device, the call raises.  torch is used only
for device memory (tensors, the caching allocator for scratch) and for the
current stream handle.
"""
import atexit
import ctypes
import os
import threading

import torch

_LIB_NAME = 'libkfac_hip.so'
_lib = None
_lock = threading.Lock()

c_int = ctypes.c_int
c_i64 = ctypes.c_int64
c_f32 = ctypes.c_float
c_ptr = ctypes.c_void_p
c_size = ctypes.c_size_t



class FactorJob(ctypes.Structure):
    """kfac_factor_job of include/kfac_hip.h: one product of kfac_factor_grouped."""
    _fields_ = [('kind', c_int), ('add_bias', c_int), ('x', c_ptr), ('rows', c_i64),
                ('c', c_int), ('H', c_int), ('W', c_int),
                ('kh', c_int), ('kw', c_int), ('sh', c_int), ('sw', c_int),
                ('ph', c_int), ('pw', c_int), ('dh', c_int), ('dw', c_int),
                ('alpha', c_f32), ('beta', c_f32), ('C_prev', c_ptr), ('C', c_ptr)]


FACTOR_LINEAR, FACTOR_CONV_A, FACTOR_CONV_G = 0, 1, 2

ERRORS = {1: 'invalid argument', 2: 'workspace too small', 3: 'HIP launch failed',
          4: 'problem too large for the built-in scratch'}


class KfacHipError(RuntimeError):
    pass


def lib_path():
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), _LIB_NAME)


_SIGNATURES = {
    'kfac_abi_version': (c_int, []),
    'kfac_factor_workspace_bytes': (c_size, [c_int, c_i64]),
    'kfac_factor_conv_a_workspace_bytes': (c_size, [c_int] * 13),
    'kfac_factor_executed_flops': (ctypes.c_double, [c_int, c_i64]),
    'kfac_factor_conv_a_executed_flops': (ctypes.c_double, [c_int] * 13),
    'kfac_factor_linear': (c_int, [c_ptr, c_i64, c_int, c_i64, c_int, c_f32, c_f32, c_ptr, c_ptr,
                                   c_ptr, c_size, c_ptr]),
    'kfac_factor_conv_a': (c_int, [c_ptr] + [c_int] * 13 + [c_f32, c_f32, c_ptr, c_ptr,
                                                           c_ptr, c_size, c_ptr]),
    'kfac_factor_conv_g': (c_int, [c_ptr, c_int, c_int, c_int, c_int, c_f32, c_f32, c_ptr, c_ptr,
                                   c_ptr, c_size, c_ptr]),
    'kfac_factor_grouped_workspace_bytes': (c_size, [c_int, c_ptr]),
    'kfac_factor_grouped_executed_flops': (ctypes.c_double, [c_int, c_ptr]),
    'kfac_inverse_executed_flops': (ctypes.c_double, [c_int, c_ptr, c_ptr]),
    'kfac_precondition_executed_flops': (ctypes.c_double, [c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    'kfac_factor_grouped': (c_int, [c_int, c_ptr, c_ptr, c_size, c_ptr]),
    'kfac_inverse_workspace_bytes': (c_size, [c_int, c_ptr]),
    'kfac_pi_damped_inverse_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr,
                                               c_ptr, c_ptr, c_ptr, c_size, c_ptr]),
    'kfac_pi_damped_inverse_std_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr,
                                                   c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_size, c_ptr]),
    'kfac_pi_damped_inverse_factored_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr,
                                                        c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr,
                                                        c_size, c_ptr]),
    'kfac_precondition_factored_workspace_bytes': (c_size, [c_int, c_ptr, c_ptr]),
    'kfac_precondition_factored_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr,
                                                   c_ptr, c_ptr, c_ptr, c_size, c_ptr]),
    'kfac_damped_inverse_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr,
                                            c_ptr, c_size, c_ptr]),
    'kfac_static_workspace_bytes': (c_size, []),
    'kfac_damped_inverse_batched_static': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr]),
    'kfac_cholesky_upper_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_ptr,
                                            c_ptr, c_size, c_ptr]),
    'kfac_precondition_workspace_bytes': (c_size, [c_int, c_ptr, c_ptr]),
    'kfac_precondition_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr,
                                          c_ptr, c_size, c_ptr]),
    'kfac_sample_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr,
                                    c_ptr, c_ptr, c_f32, c_ptr, c_size, c_ptr]),
    'kfac_vector_workspace_bytes': (c_size, [c_int]),
    'kfac_axpby_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_f32, c_f32,
                                   c_ptr, c_size, c_ptr]),
    'kfac_diag_inverse_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_int,
                                          c_ptr, c_size, c_ptr]),
    'kfac_pack_workspace_bytes': (c_size, [c_int]),
    'kfac_packed_numel': (c_i64, [c_int, c_ptr, c_ptr, c_ptr]),
    'kfac_pack_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_i64,
                                  c_ptr, c_size, c_ptr]),
    'kfac_unpack_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_i64,
                                    c_ptr, c_size, c_ptr]),
    'kfac_sqrt_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_size, c_ptr]),
    'kfac_max_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_size, c_ptr]),
    'kfac_diag_sample_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr,
                                         c_ptr, c_size, c_ptr]),
    'kfac_diag_cov_linear': (c_int, [c_ptr, c_ptr, c_int, c_int, c_int, c_int, c_f32,
                                     c_ptr, c_ptr, c_ptr]),
    'kfac_diag_cov_conv2d_workspace_bytes': (c_size, [c_int] * 5),
    'kfac_diag_cov_conv2d': (c_int, [c_ptr, c_ptr] + [c_int] * 13 + [c_f32, c_ptr,
                                                                   c_ptr, c_size, c_ptr]),
    'kfac_diag_precondition_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr,
                                               c_ptr, c_size, c_ptr]),
    'kfac_sgd_update_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr,
                                        c_ptr, c_size, c_ptr]),
    'kfac_scale_rows': (c_int, [c_ptr, c_ptr, c_i64, c_i64, c_int, c_ptr, c_ptr]),
    'kfac_rowsq_sum': (c_int, [c_ptr, c_i64, c_int, c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    'kfac_bn_diag_combine': (c_int, [c_ptr, c_ptr, c_int, c_int, c_f32, c_ptr, c_ptr, c_ptr]),
    'kfac_bn_diag_cov_workspace_bytes': (c_size, [c_int, c_int]),
    'kfac_bn_diag_cov': (c_int, [c_ptr, c_int, c_int, c_int, c_ptr, c_f32, c_ptr, c_ptr, c_ptr,
                                 c_size, c_ptr]),
    'kfac_bn_diag_cov_batched_workspace_bytes': (c_size, [c_int]),
    'kfac_bn_diag_cov_batched': (c_int, [c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr,
                                         c_ptr, c_ptr, c_size, c_ptr]),
}


def int_array(values):
    return (ctypes.c_int * len(values))(*[int(v) for v in values])


def i64_array(values):
    return (ctypes.c_int64 * len(values))(*[int(v) for v in values])


def f32_array(values):
    return (ctypes.c_float * len(values))(*[float(v) for v in values])


def ptr_array(tensors, what='tensor', allow_none=False):
    """Host array of device addresses (0 for None when allowed)."""
    out = (ctypes.c_void_p * len(tensors))()
    for i, t in enumerate(tensors):
        if t is None:
            if not allow_none:
                raise KfacHipError('%s %d is None' % (what, i))
            out[i] = None
        else:
            out[i] = dev_ptr(t, '%s %d' % (what, i))
    return out


def signatures():
    return dict(_SIGNATURES)


def load():
    """Load the shared library once; raises KfacHipError if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = lib_path()
        if not os.path.exists(path):
            raise KfacHipError(
                '%s is not built: run `python pytorch-sso_amd/build_ext.py` '
                '(there is no CPU or PyTorch fallback for the K-FAC kernels)' % path)
        lib = ctypes.CDLL(path)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(status, what):
    if status != 0:
        raise KfacHipError('%s failed: %s (code %d)' % (what, ERRORS.get(status, '?'), status))


def dev_ptr(t, what='tensor'):
    """Device address of a contiguous fp32 HIP tensor (loud otherwise)."""
    if not isinstance(t, torch.Tensor):
        raise KfacHipError('%s: expected a torch.Tensor' % what)
    if not t.is_cuda:
        raise KfacHipError('%s is on %s: the K-FAC kernels run on a HIP device only '
                           '(no CPU path exists in this package)' % (what, t.device))
    if t.dtype != torch.float32:
        raise KfacHipError('%s has dtype %s, expected float32' % (what, t.dtype))
    if not t.is_contiguous():
        raise KfacHipError('%s is not contiguous' % what)
    return t.data_ptr()


def stream_ptr(device=None, stream=None):
    """Raw handle of `stream` (a torch.cuda.Stream), or of torch's current stream."""
    if stream is not None:
        return stream.cuda_stream
    return torch.cuda.current_stream(device).cuda_stream


_all_workspaces = []     # the `bufs` dict of every thread's _Workspace


class _Workspace(threading.local):
    """Per-thread, per-device, per-stream scratch taken from torch's caching
    allocator and grown on demand (forward hooks run on the caller's thread,
    backward hooks on autograd's worker thread; each gets its own buffer, and so
    does each stream: kernels of two streams may run at the same time)."""

    def __init__(self):
        self.bufs = {}
        with _lock:
            _all_workspaces.append(self.bufs)

    def get(self, device, nbytes, stream=None):
        nbytes = int(nbytes)
        if nbytes == 0:
            return None, 0
        if device.type != 'cuda':
            raise KfacHipError('scratch requested on %s: the K-FAC kernels run on a HIP device '
                               'only (no CPU path exists in this package)' % device)
        key = (device.type, device.index, stream_ptr(device, stream))
        buf = self.bufs.get(key)
        if buf is None or buf.numel() < nbytes:
            if buf is not None and stream is not None:
                # kernels of that stream may still use the buffer that is dropped here
                buf.record_stream(stream)
            # round up so that a slowly growing request does not reallocate each time
            size = max(nbytes, 1 << 20)
            size = 1 << (size - 1).bit_length()
            buf = torch.empty(size, dtype=torch.uint8, device=device)
            self.bufs[key] = buf
        return buf, buf.numel()


_workspace = _Workspace()


def release_workspaces():
    """Drops every cached scratch buffer (all threads).  Also runs at interpreter exit, after
    a device synchronisation and before the HIP runtime and the libraries loaded beside it
    (a profiler's tool library, for one) start their own teardown: nothing of this package
    is then in flight or holds device memory while they unload."""
    with _lock:
        for bufs in _all_workspaces:
            bufs.clear()


def _at_exit():
    try:
        if _lib is not None and torch.cuda.is_initialized():
            torch.cuda.synchronize()
    except Exception:
        pass
    release_workspaces()


atexit.register(_at_exit)


def workspace(device, nbytes, stream=None):
    """(tensor-or-None, usable bytes) of the scratch of `stream` (default: torch's
    current stream); the tensor must stay referenced until the kernels using it have
    been enqueued (stream order then protects it)."""
    return _workspace.get(device, nbytes, stream)
