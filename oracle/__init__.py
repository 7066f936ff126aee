"""CPU oracle for the DDF operator.  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import
this package; the product (``ddfnet_amd``) never does and fails loudly when its
HIP library is missing.

Three independent restatements of the same operator live here so that they can
pin one another:

``loop_forward``
    Literal nested Python loops following ``grad_check.py:11-30`` of the
    reference, extended to stride with the index arithmetic of
    ``ddf/src/cuda/ddf_mul_cuda_kernel.cu:110-113``.  Tiny inputs only.
``unfold_forward``
    Vectorised ``F.unfold`` form; differentiable, so ``torch.autograd`` yields
    all three gradients without any hand-written backward formula.
``forward`` / ``backward``
    ``ddf_oracle.c`` (plain C gather loops, fp64) through ctypes; fast enough
    for the full benchmark shapes.  ``*_f32`` variants are the timed CPU
    baseline.
``up_forward`` / ``up_backward``
    The up-sampling composition of ``DDFUpPack.forward``: ``forward`` per
    sub-pixel branch, interleaved as ``F.pixel_shuffle`` would; pinned against
    ``torch.stack`` + ``F.pixel_shuffle`` of the unfold form and its autograd.

Parity status: every function here is pinned by ``tests/test_oracle.py``
(closed forms against ``F.conv2d`` / pointwise / shift, mutual agreement of
the three restatements, numerical differentiation of the forward for the
gradients, trilinearity invariants).  The reference ships no golden vectors
for this path, so none are used.
"""
import ctypes
import os
import subprocess

import numpy as np
import torch
import torch.nn.functional as F

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, 'libddf_oracle.so')
_lib = None

COMBINE = {'mul': 0, 'add': 1}


def build(force=False):
    """Compile ``ddf_oracle.c`` into ``libddf_oracle.so`` next to it."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(['make', '-s', '-C', _HERE, 'libddf_oracle.so'])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.ddf_oracle_num_threads.restype = ctypes.c_int
    return _lib


def num_threads():
    return int(lib().ddf_oracle_num_threads())


def set_num_threads(n):
    lib().ddf_oracle_set_num_threads(ctypes.c_int(int(n)))


def _np(t, dtype):
    if isinstance(t, torch.Tensor):
        t = t.detach().cpu().numpy()
    return np.ascontiguousarray(t, dtype=dtype)


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _dims(x, cf, sf, k, d, s):
    N, C, H, W = x.shape
    assert k % 2 == 1 and k >= 1 and d >= 1 and s >= 1
    assert tuple(cf.shape) == (N, C, k, k), (cf.shape, x.shape, k)
    assert tuple(sf.shape) == (N, k * k, H // s, W // s), (sf.shape, x.shape, k, s)
    return N, C, H, W


def _call(name, arrays, dims, k, d, s, combine):
    fn = getattr(lib(), name)
    args = [_ptr(a) for a in arrays] + [ctypes.c_int64(v) for v in dims] + \
        [ctypes.c_int(k), ctypes.c_int(d), ctypes.c_int(s), ctypes.c_int(COMBINE[combine])]
    fn.restype = None
    fn(*args)


def _forward(x, cf, sf, k, d, s, combine, np_dtype, suffix):
    x, cf, sf = _np(x, np_dtype), _np(cf, np_dtype), _np(sf, np_dtype)
    N, C, H, W = _dims(x, cf, sf, k, d, s)
    out = np.empty((N, C, H // s, W // s), dtype=np_dtype)
    _call('ddf_oracle_forward_' + suffix, [x, cf, sf, out], (N, C, H, W), k, d, s, combine)
    return torch.from_numpy(out)


def _backward(go, x, cf, sf, k, d, s, combine, np_dtype, suffix):
    go, x, cf, sf = (_np(a, np_dtype) for a in (go, x, cf, sf))
    N, C, H, W = _dims(x, cf, sf, k, d, s)
    assert go.shape == (N, C, H // s, W // s)
    dx, dcf, dsf = np.empty_like(x), np.empty_like(cf), np.empty_like(sf)
    dims = (N, C, H, W)
    _call('ddf_oracle_backward_features_' + suffix, [go, cf, sf, dx], dims, k, d, s, combine)
    _call('ddf_oracle_backward_channel_filter_' + suffix, [go, x, sf, dcf], dims, k, d, s, combine)
    _call('ddf_oracle_backward_spatial_filter_' + suffix, [go, x, cf, dsf], dims, k, d, s, combine)
    return torch.from_numpy(dx), torch.from_numpy(dcf), torch.from_numpy(dsf)


def forward(x, cf, sf, k=3, d=1, s=1, combine='mul'):
    """fp64 forward of the C oracle; inputs of any float dtype are widened."""
    return _forward(x, cf, sf, k, d, s, combine, np.float64, 'f64')


def backward(go, x, cf, sf, k=3, d=1, s=1, combine='mul'):
    """fp64 gradients ``(dX, dCF, dSF)`` of the C oracle."""
    return _backward(go, x, cf, sf, k, d, s, combine, np.float64, 'f64')


def forward_f32(x, cf, sf, k=3, d=1, s=1, combine='mul'):
    return _forward(x, cf, sf, k, d, s, combine, np.float32, 'f32')


def backward_f32(go, x, cf, sf, k=3, d=1, s=1, combine='mul'):
    return _backward(go, x, cf, sf, k, d, s, combine, np.float32, 'f32')


def loop_forward(x, cf, sf, k=3, d=1, s=1, combine='mul'):
    """Six nested loops, after ``grad_check.py:11-30``; stride handled as in
    ``ddf_mul_cuda_kernel.cu:110-113`` (window centred on ``y*s``, ``x*s``)."""
    x, cf, sf = (t.detach().double().cpu() for t in (x, cf, sf))
    B, C, H, W = x.shape
    Ho, Wo = H // s, W // s
    out = torch.zeros(B, C, Ho, Wo, dtype=torch.float64)
    for b in range(B):
        for c in range(C):
            for y in range(Ho):
                for xo in range(Wo):
                    acc = 0.0
                    for iy in range(k):
                        for ix in range(k):
                            yy = y * s + (iy - k // 2) * d
                            xx = xo * s + (ix - k // 2) * d
                            if yy < 0 or yy >= H or xx < 0 or xx >= W:
                                continue
                            a = float(cf[b, c, iy, ix])
                            g = float(sf[b, iy * k + ix, y, xo])
                            w = a * g if combine == 'mul' else a + g
                            acc += w * float(x[b, c, yy, xx])
                    out[b, c, y, xo] = acc
    return out


def unfold_forward(x, cf, sf, k=3, d=1, s=1, combine='mul'):
    """Vectorised, differentiable form.  ``F.unfold`` yields
    ``floor((H-1)/s)+1`` window positions per axis; the operator keeps only the
    first ``H//s`` (``ddf/ddf.py:56``, ``:74``)."""
    N, C, H, W = x.shape
    Ho, Wo = H // s, W // s
    r = (k - 1) // 2
    cols = F.unfold(x, k, dilation=d, padding=r * d, stride=s)
    hu, wu = (H - 1) // s + 1, (W - 1) // s + 1
    cols = cols.view(N, C, k * k, hu, wu)[:, :, :, :Ho, :Wo]
    a = cf.reshape(N, C, k * k, 1, 1)
    b = sf.reshape(N, 1, k * k, Ho, Wo)
    w = a * b if combine == 'mul' else a + b
    return (cols * w).sum(dim=2)


def unfold_backward(go, x, cf, sf, k=3, d=1, s=1, combine='mul'):
    """Gradients by autograd through ``unfold_forward``."""
    x, cf, sf = (t.detach().clone().requires_grad_(True) for t in (x, cf, sf))
    out = unfold_forward(x, cf, sf, k, d, s, combine)
    return torch.autograd.grad(out, (x, cf, sf), go)


def up_forward(x, cfs, sfs, k=3, d=1, scale=2, combine='mul'):
    """Up-sampling DDF as ``DDFUpPack.forward`` composes it
    (``ddf/ddf.py:264-272``): one stride-1 ``forward`` per sub-pixel branch
    ``b = i*scale + j``, whose result lands on the pixels ``(y*scale + i,
    x*scale + j)`` -- what ``torch.stack(outs, 2)`` + ``F.pixel_shuffle`` do."""
    N, C, H, W = x.shape
    out = torch.zeros(N, C, H * scale, W * scale, dtype=torch.float64)
    for b, (cf, sf) in enumerate(zip(cfs, sfs)):
        i, j = divmod(b, scale)
        out[:, :, i::scale, j::scale] = forward(x, cf, sf, k, d, 1, combine)
    return out


def up_backward(go, x, cfs, sfs, k=3, d=1, scale=2, combine='mul'):
    """Gradients of ``up_forward``: ``(dX, [dCF_b], [dSF_b])``.  Branch ``b``
    sees the gradient of its own sub-pixel lattice; dX sums over branches."""
    dx, dcfs, dsfs = 0, [], []
    for b, (cf, sf) in enumerate(zip(cfs, sfs)):
        i, j = divmod(b, scale)
        g = go[:, :, i::scale, j::scale].contiguous()
        dxb, dcf, dsf = backward(g, x, cf, sf, k, d, 1, combine)
        dx = dx + dxb
        dcfs.append(dcf)
        dsfs.append(dsf)
    return dx, dcfs, dsfs


def filter_standardize(f, dim):
    """``(f - mean) / (std_unbiased + 1e-10)`` over ``dim``: the core of
    ``FilterNorm.forward`` (``ddf/ddf.py:149-150``, ``:162-163``) with no gain."""
    f = f - f.mean(dim=dim, keepdim=True)
    return f / (f.std(dim=dim, keepdim=True) + 1e-10)


def make_inputs(N, C, H, W, k=3, s=1, dtype=torch.float32, standardize=True, seed=0):
    """Seeded benchmark inputs: features, channel filter, spatial filter and
    grad-output drawn in that order from N(0,1) on the CPU generator; filters
    optionally standardised over their taps; then cast to ``dtype``."""
    g = torch.Generator(device='cpu').manual_seed(seed)
    base = torch.float64 if dtype == torch.float64 else torch.float32
    Ho, Wo = H // s, W // s
    x = torch.randn(N, C, H, W, generator=g, dtype=base)
    cf = torch.randn(N, C, k, k, generator=g, dtype=base)
    sf = torch.randn(N, k * k, Ho, Wo, generator=g, dtype=base)
    go = torch.randn(N, C, Ho, Wo, generator=g, dtype=base)
    if standardize and k > 1:
        cf = filter_standardize(cf.reshape(N, C, k * k), 2).reshape(N, C, k, k)
        sf = filter_standardize(sf, 1)
    return tuple(t.to(dtype).contiguous() for t in (x, cf, sf, go))
