"""ddf_hip_backward_spatial_norm: the operator's backward pass with the spatial
branch's filter normalisation behind it (FilterNorm 'spatial' in front of ddf,
ddf/ddf.py:146-157 and :217-221 of the reference).

Called through the C ABI and through the autograd node built on it, and held to
the fp64 CPU composition: oracle backward for dX / dCF / dSF, then the gradient
of gain * (raw - mean) / (std + 1e-10) by torch autograd."""
import ctypes

import pytest
import torch

import oracle
from ddfnet_amd import _lib, functional
from ddf_testlib import TOL, rel_err

pytestmark = pytest.mark.gpu


def _normalise(raw, groups, gain, gain_vec):
    """(N, kk, Ho, Wo) -> gain * standardised over the taps; sample n uses gain_vec row n % groups."""
    n, kk = raw.shape[:2]
    var, mean = torch.var_mean(raw, dim=1, keepdim=True)
    z = (raw - mean) / (var.sqrt() + 1e-10)
    if gain_vec is None:
        return z * gain, z
    w = gain_vec.view(groups, kk)[torch.arange(n) % groups].view(n, kk, 1, 1)
    return z * w, z


def _case(shape, k, s, dtype, groups, learned, seed):
    N, C, H, W = shape
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(N, C, H, W, generator=g).to(dtype)
    cf = torch.randn(N, C, k, k, generator=g).to(dtype)
    raw = (torch.randn(N, k * k, H // s, W // s, generator=g) * 1.5 + 0.3).to(dtype)
    go = torch.randn(N, C, H // s, W // s, generator=g).to(dtype)
    gain_vec = (torch.randn(groups * k * k, generator=g) * 0.5 + 0.6).to(dtype) if learned else None
    return x, cf, raw, go, gain_vec


def _expected(x, cf, raw, go, gain_vec, k, d, s, combine, groups, gain, sf_used):
    """fp64 on the rounded inputs; the operator's part with the normalised filter the
    GPU forward pass really used (sf_used, rounded to the storage type)."""
    rawd = raw.double().requires_grad_(True)
    gv = None if gain_vec is None else gain_vec.double().requires_grad_(True)
    sf, z = _normalise(rawd, groups, gain, gv)
    dx, dcf, dsf = oracle.backward(go, x, cf, sf_used, k, d, s, combine)
    wanted = [rawd] + ([gv] if gv is not None else [])
    grads = torch.autograd.grad(sf, wanted, dsf)
    return dx, dcf, grads[0], (grads[1] if gv is not None else None), sf.detach()


# (what each case is there for; the launches it makes are checked below)
CASES = [
    # shape, k, d, s, combine, dtype, groups, learned gain
    ((8, 64, 14, 14), 3, 1, 1, 'mul', torch.float32, 1, False),    # dSF partial sums over channel splits
    ((8, 64, 14, 14), 3, 1, 1, 'add', torch.float16, 4, True),
    ((2, 16, 56, 56), 3, 1, 1, 'mul', torch.float16, 1, False),    # complete dSF + dCF partial sums over strips
    ((2, 16, 56, 56), 3, 1, 1, 'add', torch.float32, 2, True),
    ((2, 8, 12, 12), 3, 1, 1, 'mul', torch.float32, 1, False),     # no partial sums: normalisation launch of its own
    ((4, 32, 28, 28), 3, 1, 2, 'mul', torch.float32, 2, False),    # stride 2
    ((4, 32, 28, 28), 3, 2, 1, 'mul', torch.float32, 1, True),     # dilation 2: dX and filters as two launches
    ((2, 24, 28, 28), 5, 2, 1, 'mul', torch.float32, 1, False),    # 25 taps
    ((2, 24, 20, 20), 5, 1, 1, 'add', torch.float16, 2, True),
    ((2, 6, 11, 13), 7, 1, 1, 'mul', torch.float32, 1, False),     # 49 taps: generic kernels
    ((2, 6, 9, 10), 3, 1, 1, 'mul', torch.float64, 2, True),       # fp64
    ((3, 5, 9, 7), 3, 1, 2, 'add', torch.float32, 3, False),       # odd sizes under stride 2
]


@pytest.mark.parametrize('shape,k,d,s,combine,dtype,groups,learned', CASES)
def test_backward_spatial_norm_through_the_c_abi(shape, k, d, s, combine, dtype, groups, learned):
    N, C, H, W = shape
    gain = 0.47
    x, cf, raw, go, gain_vec = _case(shape, k, s, dtype, groups, learned, seed=31)
    xd, cfd, rawd, god = (t.cuda() for t in (x, cf, raw, go))
    gvd = None if gain_vec is None else gain_vec.cuda()
    sfd = _lib.filter_norm(rawd, N // groups, groups, k * k, (H // s) * (W // s), gain, gvd)
    lib = _lib.lib()
    p = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())
    tail = (N, C, H, W, k, d, s, _lib.COMBINE[combine], _lib.DTYPE[dtype])
    need = 7
    nbytes = lib.ddf_hip_backward_spatial_norm_workspace_bytes(*tail, need, 0)
    assert nbytes >= rawd.numel() * rawd.element_size()
    ws = torch.empty(nbytes, dtype=torch.uint8, device='cuda')
    dx = torch.full_like(xd, float('nan'))
    dcf = torch.full_like(cfd, float('nan'))
    draw = torch.full_like(rawd, float('nan'))
    terms = torch.full_like(rawd, float('nan')) if learned else None
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.ddf_hip_backward_spatial_norm(p(god), p(xd), p(cfd), p(sfd), p(rawd), p(dx), p(dcf), p(draw),
                                           p(terms), p(ws), nbytes, *tail, need, groups, gain, p(gvd), 0,
                                           stream)
    assert rc == 0, lib.ddf_hip_last_error()
    torch.cuda.synchronize()
    want_dx, want_dcf, want_draw, want_gain, _ = _expected(
        x, cf, raw, go, gain_vec, k, d, s, combine, groups, gain, sfd.cpu())
    tol = max(TOL[dtype], 1e-10) * (4 if dtype != torch.float64 else 1)   # (two roundings in a row)
    assert rel_err(dx, want_dx) <= tol
    assert rel_err(dcf, want_dcf) <= tol
    assert rel_err(draw, want_draw) <= tol
    if learned:
        got_gain = terms.double().view(N // groups, groups, k * k, -1).sum(dim=(0, 3)).reshape(-1)
        assert rel_err(got_gain, want_gain) <= tol * 4
    # where the backward pass ends with a partial-sum launch, the normalisation rides on it
    names = _lib.describe(shape, k, d, s, combine, dtype, need | 8)
    has_sum_launch = 'k_sum_partials' in _lib.describe(shape, k, d, s, combine, dtype, need)
    if has_sum_launch and k in (3, 5):
        assert 'k_sum_norm_pair' in names and 'k_filter_norm_backward' not in names, names
    else:
        assert names.endswith('k_filter_norm_backward'), names
    # a workspace that is too small is refused before anything is launched
    rc = lib.ddf_hip_backward_spatial_norm(p(god), p(xd), p(cfd), p(sfd), p(rawd), p(dx), p(dcf), p(draw),
                                           p(terms), p(ws), nbytes - 256, *tail, need, groups, gain, p(gvd),
                                           0, stream)
    assert rc == 3
    # groups must divide N
    rc = lib.ddf_hip_backward_spatial_norm(p(god), p(xd), p(cfd), p(sfd), p(rawd), p(dx), p(dcf), p(draw),
                                           p(terms), p(ws), nbytes, *tail, need, N + 1, gain, p(gvd), 0,
                                           stream)
    assert rc == 1


@pytest.mark.parametrize('shape,k,d,s,combine,dtype,groups,learned', CASES[:4] + CASES[5:6])
def test_autograd_node_equals_norm_then_operator(shape, k, d, s, combine, dtype, groups, learned):
    """ddf_spatial_norm against FilterNorm's launch followed by ddf: same forward
    bits, gradients within rounding (the fused route keeps dSF in fp32 on its way
    through the normalisation)."""
    from ddfnet_amd import ddf, modules
    N, C, H, W = shape
    gain = 0.47
    x, cf, raw, go, gain_vec = _case(shape, k, s, dtype, groups, learned, seed=32)

    def leaves():
        ts = [t.cuda().requires_grad_(True) for t in (x, cf, raw)]
        gv = None if gain_vec is None else gain_vec.cuda().requires_grad_(True)
        return ts, gv

    (xa, cfa, rawa), gva = leaves()
    out_a = functional.ddf_spatial_norm(xa, cfa, rawa, k, d, s, combine, groups, gain, gva)
    (xb, cfb, rawb), gvb = leaves()
    sf = modules._FilterNormFunction.apply(rawb, gvb, None, N // groups, groups, k * k,
                                           (H // s) * (W // s), gain)
    out_b = ddf(xb, cfb, sf, k, d, s, combine)
    assert torch.equal(out_a, out_b)
    la = [xa, cfa, rawa] + ([gva] if learned else [])
    lb = [xb, cfb, rawb] + ([gvb] if learned else [])
    ga = torch.autograd.grad(out_a, la, go.cuda())
    gb = torch.autograd.grad(out_b, lb, go.cuda())
    tol = 2e-5 if dtype == torch.float32 else 1e-2
    for name, u, v in zip(('dX', 'dCF', 'dRaw', 'dGain'), ga, gb):
        assert rel_err(u, v.detach().cpu()) <= tol, name
    # only what autograd asks for
    (xa, cfa, rawa), gva = leaves()
    out = functional.ddf_spatial_norm(xa.detach(), cfa.detach(), rawa, k, d, s, combine, groups, gain,
                                      None if gva is None else gva.detach())
    (g_raw,) = torch.autograd.grad(out, [rawa], go.cuda())
    assert rel_err(g_raw, ga[2].detach().cpu()) <= tol
