"""ctypes binding of ``libddf_hip.so`` (declared in ``include/ddf_hip.h``).

torch is imported before the library is opened so that both share one HIP
runtime; torch is used only to obtain device pointers and the current stream.
There is no CPU fallback: a missing library raises.
"""
import ctypes
import os

import torch  # noqa: F401  (must load its HIP runtime first)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'libddf_hip.so')

DTYPE = {torch.float16: 0, torch.float32: 1, torch.float64: 2}
COMBINE = {'mul': 0, 'add': 1}
VARIANT = {'': 0, 'o': 1, 'f': 2}
NEED_DX, NEED_DCF, NEED_DSF = 1, 2, 4

# name -> (restype, argtypes); must list every symbol of include/ddf_hip.h
_vp, _i64, _i, _u, _sz = (ctypes.c_void_p, ctypes.c_int64, ctypes.c_int,
                          ctypes.c_uint, ctypes.c_size_t)
SYMBOLS = {
    'ddf_hip_version': (_i, []),
    'ddf_hip_status_string': (ctypes.c_char_p, [_i]),
    'ddf_hip_last_error': (ctypes.c_char_p, []),
    'ddf_hip_forward': (_i, [_vp] * 4 + [_i64] * 4 + [_i] * 6 + [_vp]),
    'ddf_hip_backward_workspace_bytes': (_sz, [_i64] * 4 + [_i] * 5 + [_u, _i]),
    'ddf_hip_backward': (_i, [_vp] * 8 + [_sz] + [_i64] * 4 + [_i] * 5 + [_u, _i, _vp]),
}

_lib = None


class DDFHipError(RuntimeError):
    pass


def is_built():
    return os.path.exists(LIB_PATH)


def lib():
    """Open the library once.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not is_built():
            raise DDFHipError(
                'HIP library %s is missing; build it with `python -m ddfnet_amd.build` '
                '(there is no CPU or PyTorch fallback for the ddf operator)' % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


def check(status):
    if status != 0:
        l = lib()
        raise DDFHipError('%s: %s' % (l.ddf_hip_status_string(status).decode(),
                                      l.ddf_hip_last_error().decode()))


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def forward(features, channel_filter, spatial_filter, output, k, d, s, combine, variant=''):
    """Enqueue the forward kernels on torch's current stream.  Tensors must be
    contiguous device tensors of one dtype, on the current device."""
    N, C, H, W = features.shape
    check(lib().ddf_hip_forward(
        _ptr(features), _ptr(channel_filter), _ptr(spatial_filter), _ptr(output),
        N, C, H, W, k, d, s, COMBINE[combine], DTYPE[features.dtype], VARIANT[variant],
        _stream()))


def backward_workspace_bytes(shape, k, d, s, combine, dtype, need, variant=''):
    N, C, H, W = shape
    return int(lib().ddf_hip_backward_workspace_bytes(
        N, C, H, W, k, d, s, COMBINE[combine], DTYPE[dtype], need, VARIANT[variant]))


def backward(grad_output, features, channel_filter, spatial_filter, grad_features,
             grad_channel_filter, grad_spatial_filter, k, d, s, combine, need,
             workspace=None, variant=''):
    N, C, H, W = features.shape
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    check(lib().ddf_hip_backward(
        _ptr(grad_output), _ptr(features), _ptr(channel_filter), _ptr(spatial_filter),
        _ptr(grad_features), _ptr(grad_channel_filter), _ptr(grad_spatial_filter),
        _ptr(workspace), ws_bytes, N, C, H, W, k, d, s, COMBINE[combine],
        DTYPE[features.dtype], need, VARIANT[variant], _stream()))
