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
ERR_UNSUPPORTED = 2   # DDF_ERR_UNSUPPORTED

# name -> (restype, argtypes); must list every symbol of include/ddf_hip.h
_vp, _i64, _i, _u, _sz = (ctypes.c_void_p, ctypes.c_int64, ctypes.c_int,
                          ctypes.c_uint, ctypes.c_size_t)
SYMBOLS = {
    'ddf_hip_version': (_i, []),
    'ddf_hip_status_string': (ctypes.c_char_p, [_i]),
    'ddf_hip_last_error': (ctypes.c_char_p, []),
    'ddf_hip_describe': (_i, [_i64] * 4 + [_i] * 5 + [_u, _i, ctypes.c_char_p, _i]),
    'ddf_hip_forward': (_i, [_vp] * 4 + [_i64] * 4 + [_i] * 6 + [_vp]),
    'ddf_hip_backward_workspace_bytes': (_sz, [_i64] * 4 + [_i] * 5 + [_u, _i]),
    'ddf_hip_backward': (_i, [_vp] * 8 + [_sz] + [_i64] * 4 + [_i] * 5 + [_u, _i, _vp]),
    'ddf_hip_backward_static': (_i, [_vp] * 7 + [_i64] * 4 + [_i] * 5 + [_u, _i, _vp]),
    'ddf_hip_backward_spatial_norm_workspace_bytes': (_sz, [_i64] * 4 + [_i] * 5 + [_u, _i]),
    'ddf_hip_backward_spatial_norm': (_i, [_vp] * 10 + [_sz] + [_i64] * 4 + [_i] * 5 +
                                      [_u, _i, ctypes.c_double, _vp, _i, _vp]),
    'ddf_hip_filter_norm': (_i, [_vp] * 2 + [_i64] * 2 + [_i, _i64, ctypes.c_double] + [_vp] * 2 +
                            [_i, _vp]),
    'ddf_hip_filter_norm_backward': (_i, [_vp] * 4 + [_i64] * 2 + [_i, _i64, ctypes.c_double, _vp,
                                          _i, _vp]),
    'ddf_hip_spatial_branch': (_i, [_vp] * 4 + [_i64] * 4 + [_i] * 3 + [ctypes.c_double] +
                               [_vp] * 2 + [_i, _vp]),
    'ddf_hip_channel_branch': (_i, [_vp] * 6 + [_i64] * 3 + [_i, ctypes.c_double] + [_vp] * 2 +
                               [_i, _vp]),
    'ddf_hip_spatial_branch_pool': (_i, [_vp] * 5 + [_i64, ctypes.POINTER(ctypes.c_int)] + [_i64] * 4 +
                                    [_i] * 3 + [ctypes.c_double] + [_vp] * 2 + [_i, _vp]),
    'ddf_hip_channel_branch_parts': (_i, [_vp, _i, ctypes.c_double] + [_vp] * 5 + [_i64] * 3 +
                                     [_i, ctypes.c_double] + [_vp] * 2 + [_i, _vp]),
    'ddf_hip_up_forward': (_i, [_vp] * 4 + [_i64] * 4 + [_i] * 5 + [_vp]),
    'ddf_hip_up_backward_workspace_bytes': (_sz, [_i64] * 4 + [_i] * 5 + [_u]),
    'ddf_hip_up_backward': (_i, [_vp] * 8 + [_sz] + [_i64] * 4 + [_i] * 5 + [_u, _vp]),
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


_raw_stream = getattr(torch._C, '_cuda_getCurrentRawStream', None)


def _stream():
    """torch's current stream on the current device, as a hipStream_t."""
    if _raw_stream is not None:   # same value, without building a Stream object
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


class on_device_of(object):
    """Device guard that costs nothing when the tensor already lives on the
    current device (the common case)."""

    def __init__(self, tensor):
        idx = tensor.device.index
        self.guard = None if idx == torch.cuda.current_device() else torch.cuda.device(idx)

    def __enter__(self):
        if self.guard is not None:
            self.guard.__enter__()

    def __exit__(self, *exc):
        if self.guard is not None:
            self.guard.__exit__(*exc)
        return False


def describe(shape, k, d, s, combine, dtype, need=0, variant=''):
    """Names of the kernels a forward (need = 0) or backward call launches."""
    N, C, H, W = shape
    buf = ctypes.create_string_buffer(256)
    check(lib().ddf_hip_describe(N, C, H, W, k, d, s, COMBINE[combine], DTYPE[dtype], need,
                                 VARIANT[variant], buf, len(buf)))
    return buf.value.decode()


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


def backward_spatial_norm(grad_output, features, channel_filter, spatial_filter, raw_spatial_filter,
                          grad_features, grad_channel_filter, grad_raw_spatial_filter, gain_terms,
                          k, d, s, combine, need, groups, gain, gain_vec=None, variant=''):
    """``backward`` with the spatial filter normalisation behind dSF: writes the
    gradient with respect to the raw (un-normalised) spatial filter.  Allocates
    its workspace from torch's caching allocator."""
    N, C, H, W = features.shape
    tail = (N, C, H, W, k, d, s, COMBINE[combine], DTYPE[features.dtype])
    nbytes = lib().ddf_hip_backward_spatial_norm_workspace_bytes(*tail, need, VARIANT[variant])
    workspace = (torch.empty(nbytes, dtype=torch.uint8, device=features.device) if nbytes else None)
    check(lib().ddf_hip_backward_spatial_norm(
        _ptr(grad_output), _ptr(features), _ptr(channel_filter), _ptr(spatial_filter),
        _ptr(raw_spatial_filter), _ptr(grad_features), _ptr(grad_channel_filter),
        _ptr(grad_raw_spatial_filter), _ptr(gain_terms), _ptr(workspace), nbytes, *tail, need,
        groups, float(gain), _ptr(gain_vec), VARIANT[variant], _stream()))


def filter_norm(x, outer, groups, taps, inner, gain, gain_vec=None, offset_vec=None):
    """y = gain * standardised(x) + offset over the taps of a contiguous
    (outer, groups, taps, inner) device tensor; returns a new tensor shaped
    like ``x``.  Enqueued on torch's current stream."""
    y = torch.empty_like(x)
    with on_device_of(x):
        rc = lib().ddf_hip_filter_norm(
            _ptr(x), _ptr(y), outer, groups, taps, inner, float(gain), _ptr(gain_vec),
            _ptr(offset_vec), DTYPE[x.dtype], _stream())
    check(rc)
    return y


def filter_norm_backward(grad_y, x, outer, groups, taps, inner, gain, gain_vec=None,
                         want_gain_terms=False):
    """Gradient of ``filter_norm`` with respect to ``x``; also returns
    ``grad_y * standardised(x)`` (or None), whose sum over (outer, inner) is
    the gradient of ``gain_vec``."""
    grad_x = torch.empty_like(x)
    terms = torch.empty_like(x) if want_gain_terms else None
    with on_device_of(x):
        rc = lib().ddf_hip_filter_norm_backward(
            _ptr(grad_y), _ptr(x), _ptr(grad_x), _ptr(terms), outer, groups, taps, inner,
            float(gain), _ptr(gain_vec), DTYPE[x.dtype], _stream())
    check(rc)
    return grad_x, terms


def spatial_branch(features, weight, bias, head, k, stride, gain, gain_vec=None, offset_vec=None):
    """1x1 convolution (stride as the operator's) + spatial filter normalisation
    in one launch; returns the (N, head*k*k, H//stride, W//stride) taps."""
    N, C, H, W = features.shape
    sf = features.new_empty((N, head * k * k, H // stride, W // stride))
    with on_device_of(features):
        rc = lib().ddf_hip_spatial_branch(
            _ptr(features), _ptr(weight), _ptr(bias), _ptr(sf), N, C, H, W, head, k, stride,
            float(gain), _ptr(gain_vec), _ptr(offset_vec), DTYPE[features.dtype], _stream())
    check(rc)
    return sf


def channel_branch(pooled, weight1, bias1, weight2, bias2, k, gain, gain_vec=None,
                   offset_vec=None):
    """Bottleneck MLP on the pooled (N, C) features + channel filter
    normalisation in one launch; returns the (N, C, k, k) filters."""
    N, C = pooled.shape
    mid = weight1.shape[0]
    cf = pooled.new_empty((N, C, k, k))
    with on_device_of(pooled):
        rc = lib().ddf_hip_channel_branch(
            _ptr(pooled), _ptr(weight1), _ptr(bias1), _ptr(weight2), _ptr(bias2), _ptr(cf), N, C,
            mid, k, float(gain), _ptr(gain_vec), _ptr(offset_vec), DTYPE[pooled.dtype], _stream())
    check(rc)
    return cf


def spatial_branch_pool(features, weight, bias, head, k, stride, gain, gain_vec=None, offset_vec=None):
    """spatial_branch that also leaves partial sums of every feature plane (what the
    global average pool in front of the channel branch needs); returns
    (taps, parts) with parts an fp32 (N, tiles, C) tensor, or None where the
    library has no kernel for it (then pool and call the plain entry points)."""
    N, C, H, W = features.shape
    ho, wo = H // stride, W // stride
    if N * C * ho * wo * head == 0:
        return None
    sf = features.new_empty((N, head * k * k, ho, wo))
    cap_tiles = (ho * wo + 63) // 64 * 4
    parts = torch.empty((N * cap_tiles * C,), dtype=torch.float32, device=features.device)
    nparts = ctypes.c_int(0)
    with on_device_of(features):
        rc = lib().ddf_hip_spatial_branch_pool(
            _ptr(features), _ptr(weight), _ptr(bias), _ptr(sf), _ptr(parts), parts.numel(),
            ctypes.byref(nparts), N, C, H, W, head, k, stride, float(gain), _ptr(gain_vec),
            _ptr(offset_vec), DTYPE[features.dtype], _stream())
    if rc == ERR_UNSUPPORTED:
        return None
    check(rc)
    return sf, parts[:N * nparts.value * C].view(N, nparts.value, C)


def channel_branch_parts(parts, scale, weight1, bias1, weight2, bias2, k, gain, gain_vec=None,
                         offset_vec=None):
    """channel_branch on pooled = scale * parts.sum(1), parts an fp32 (N, tiles, C)
    tensor as spatial_branch_pool returns it; the filters come out in the
    weights' dtype."""
    N, nparts, C = parts.shape
    mid = weight1.shape[0]
    cf = weight1.new_empty((N, C, k, k))
    with on_device_of(parts):
        rc = lib().ddf_hip_channel_branch_parts(
            _ptr(parts), nparts, float(scale), _ptr(weight1), _ptr(bias1), _ptr(weight2), _ptr(bias2),
            _ptr(cf), N, C, mid, k, float(gain), _ptr(gain_vec), _ptr(offset_vec),
            DTYPE[weight1.dtype], _stream())
    check(rc)
    return cf


def branches_cover(k, dtype):
    """(kernel_size, dtype) pairs the two branch kernels are built for."""
    return k in (3, 5) and dtype in (torch.float16, torch.float32)


def up_forward(features, channel_filters, spatial_filters, output, k, d, scale, combine):
    """All ``scale*scale`` sub-pixel branches of an up-sampling DDF in one
    launch; ``output`` is the pixel-shuffled (N, C, H*scale, W*scale) result.
    Raises ``DDFHipError`` when the library does not cover (k, scale)."""
    N, C, H, W = features.shape
    branches = scale * scale
    assert len(channel_filters) == branches and len(spatial_filters) == branches
    cf = (ctypes.c_void_p * branches)(*[t.data_ptr() for t in channel_filters])
    sf = (ctypes.c_void_p * branches)(*[t.data_ptr() for t in spatial_filters])
    check(lib().ddf_hip_up_forward(
        _ptr(features), cf, sf, _ptr(output), N, C, H, W, k, d, scale, COMBINE[combine],
        DTYPE[features.dtype], _stream()))


def up_backward(grad_output, features, channel_filters, spatial_filters, grad_features,
                grad_channel_filters, grad_spatial_filters, k, d, scale, combine):
    """Gradients of ``up_forward``; a gradient tensor given as None is not
    computed.  Allocates the library's workspace from torch's allocator."""
    N, C, H, W = features.shape
    branches = scale * scale
    need = ((NEED_DX if grad_features is not None else 0) |
            (NEED_DCF if any(t is not None for t in grad_channel_filters) else 0) |
            (NEED_DSF if any(t is not None for t in grad_spatial_filters) else 0))
    if need == 0:
        return

    def ptrs(tensors):
        return (ctypes.c_void_p * branches)(*[None if t is None else t.data_ptr() for t in tensors])

    dt = DTYPE[features.dtype]
    nbytes = int(lib().ddf_hip_up_backward_workspace_bytes(N, C, H, W, k, d, scale,
                                                           COMBINE[combine], dt, need))
    workspace = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=features.device)
    check(lib().ddf_hip_up_backward(
        _ptr(grad_output), _ptr(features), ptrs(channel_filters), ptrs(spatial_filters),
        _ptr(grad_features), ptrs(grad_channel_filters), ptrs(grad_spatial_filters),
        _ptr(workspace), nbytes, N, C, H, W, k, d, scale, COMBINE[combine], dt, need, _stream()))


def up_forward_covers(k, scale):
    """(kernel_size, scale) pairs ddf_hip_up_forward has kernels for."""
    return (k in (1, 3) and 2 <= scale <= 4) or (k == 5 and scale == 2)
