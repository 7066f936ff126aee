"""Pins the CPU oracle (oracle/) without the reference, which ships no golden
vectors for the operator: closed forms a library routine computes, mutual
agreement of three independently written restatements, numerical
differentiation of the forward for every gradient, and the trilinearity
invariants of the op.  Each check is chosen so that a dropped term, a flipped
tap index, a transposed (i, j) or a ceil-instead-of-floor output size fails."""
import itertools

import pytest
import torch
import torch.nn.functional as F

import oracle

torch.manual_seed(1234)

KDS = [(3, 1, 1), (3, 2, 1), (3, 1, 2), (3, 2, 2), (5, 1, 1), (5, 2, 1),
       (5, 1, 2), (5, 2, 2), (1, 1, 1), (1, 1, 2), (7, 1, 1), (3, 3, 3)]


def rand_case(N, C, H, W, k, s, dtype=torch.float64):
    x = torch.randn(N, C, H, W, dtype=dtype)
    cf = torch.randn(N, C, k, k, dtype=dtype)
    sf = torch.randn(N, k * k, H // s, W // s, dtype=dtype)
    go = torch.randn(N, C, H // s, W // s, dtype=dtype)
    return x, cf, sf, go


@pytest.mark.parametrize('combine', ['mul', 'add'])
@pytest.mark.parametrize('k,d,s', KDS)
def test_c_forward_matches_loop_and_unfold(k, d, s, combine):
    # non-square, odd sizes: H % s != 0 exercises floor(H/s)
    x, cf, sf, _ = rand_case(2, 3, 9, 11, k, s)
    ref = oracle.loop_forward(x, cf, sf, k, d, s, combine)
    assert ref.shape == (2, 3, 9 // s, 11 // s)
    got_c = oracle.forward(x, cf, sf, k, d, s, combine)
    got_u = oracle.unfold_forward(x, cf, sf, k, d, s, combine)
    assert torch.allclose(got_c, ref, rtol=0, atol=1e-12)
    assert torch.allclose(got_u, ref, rtol=0, atol=1e-12)


@pytest.mark.parametrize('k,d,s', [(3, 1, 1), (3, 2, 1), (3, 1, 2), (5, 2, 2), (5, 1, 1)])
def test_forward_reduces_to_depthwise_conv(k, d, s):
    """mul with SF == 1 (add with SF == 0) is a per-sample depthwise
    convolution (reference README.md:49-63)."""
    N, C, H, W = 2, 5, 12, 10
    x, cf, sf, _ = rand_case(N, C, H, W, k, s)
    r = (k - 1) // 2
    conv = F.conv2d(x.view(1, N * C, H, W), cf.view(N * C, 1, k, k), padding=r * d,
                    dilation=d, stride=s, groups=N * C).view(N, C, (H - 1) // s + 1, -1)
    conv = conv[:, :, :H // s, :W // s]
    assert torch.allclose(oracle.forward(x, cf, torch.ones_like(sf), k, d, s, 'mul'), conv, atol=1e-12)
    assert torch.allclose(oracle.forward(x, cf, torch.zeros_like(sf), k, d, s, 'add'), conv, atol=1e-12)


def test_forward_one_hot_is_shift():
    """CF == 1 and SF one-hot at tap (i, j) gives X shifted by ((i-r)d, (j-r)d)
    with zero fill; catches transposed or flipped tap indexing."""
    N, C, H, W, k, d = 1, 2, 8, 9, 3, 2
    x = torch.randn(N, C, H, W, dtype=torch.float64)
    cf = torch.ones(N, C, k, k, dtype=torch.float64)
    for i, j in itertools.product(range(k), range(k)):
        sf = torch.zeros(N, k * k, H, W, dtype=torch.float64)
        sf[:, i * k + j] = 1
        dy, dx = (i - 1) * d, (j - 1) * d
        want = torch.zeros_like(x)
        ys = slice(max(0, -dy), min(H, H - dy))
        xs = slice(max(0, -dx), min(W, W - dx))
        want[:, :, ys, xs] = x[:, :, ys.start + dy:ys.stop + dy, xs.start + dx:xs.stop + dx]
        assert torch.equal(oracle.forward(x, cf, sf, k, d, 1, 'mul'), want)


def test_forward_k1_is_pointwise():
    x, cf, sf, _ = rand_case(2, 3, 7, 9, 1, 2)
    sub = x[:, :, ::2, ::2][:, :, :3, :4]
    assert torch.allclose(oracle.forward(x, cf, sf, 1, 1, 2, 'mul'), sub * cf * sf, atol=1e-14)
    assert torch.allclose(oracle.forward(x, cf, sf, 1, 1, 2, 'add'), sub * (cf + sf), atol=1e-14)


@pytest.mark.parametrize('k,d,s', [(3, 1, 1), (5, 2, 2)])
def test_add_is_sum_of_two_muls(k, d, s):
    x, cf, sf, _ = rand_case(2, 4, 10, 10, k, s)
    a = oracle.forward(x, cf, torch.ones_like(sf), k, d, s, 'mul')
    b = oracle.forward(x, torch.ones_like(cf), sf, k, d, s, 'mul')
    assert torch.allclose(oracle.forward(x, cf, sf, k, d, s, 'add'), a + b, atol=1e-12)


@pytest.mark.parametrize('combine', ['mul', 'add'])
@pytest.mark.parametrize('k,d,s', KDS)
def test_c_backward_matches_autograd(k, d, s, combine):
    x, cf, sf, go = rand_case(2, 3, 9, 11, k, s)
    want = oracle.unfold_backward(go, x, cf, sf, k, d, s, combine)
    got = oracle.backward(go, x, cf, sf, k, d, s, combine)
    for g, w, name in zip(got, want, ('dX', 'dCF', 'dSF')):
        assert g.shape == w.shape
        assert torch.allclose(g, w, rtol=0, atol=1e-11), name


@pytest.mark.parametrize('combine', ['mul', 'add'])
@pytest.mark.parametrize('k,d,s', [(3, 1, 1), (3, 2, 2), (5, 2, 1), (5, 1, 2)])
def test_c_backward_matches_numerical_derivative(k, d, s, combine):
    """Central differences of the C forward; the op is multilinear, so they are
    exact up to rounding.  Independent of any backward formula."""
    x, cf, sf, go = rand_case(1, 2, 6, 7, k, s)
    got = oracle.backward(go, x, cf, sf, k, d, s, combine)
    eps = 1e-3
    tensors = [x, cf, sf]
    for which, g in enumerate(got):
        base = tensors[which]
        num = torch.zeros_like(base)
        flat, nflat = base.view(-1), num.view(-1)
        for e in range(flat.numel()):
            old = flat[e].item()
            flat[e] = old + eps
            fp = (oracle.forward(*tensors, k, d, s, combine) * go).sum()
            flat[e] = old - eps
            fm = (oracle.forward(*tensors, k, d, s, combine) * go).sum()
            flat[e] = old
            nflat[e] = (fp - fm) / (2 * eps)
        assert torch.allclose(g, num, rtol=0, atol=1e-8), which


@pytest.mark.parametrize('k,d,s', [(3, 1, 1), (3, 1, 2), (5, 2, 1)])
def test_gradient_invariants(k, d, s):
    """mul is trilinear: <dX,X> = <dCF,CF> = <dSF,SF> = <dO,O>.
    add: <dX,X> = <dO,O> and <dCF,CF> + <dSF,SF> = <dO,O>."""
    x, cf, sf, go = rand_case(2, 5, 12, 12, k, s)
    for combine in ('mul', 'add'):
        o = oracle.forward(x, cf, sf, k, d, s, combine)
        dx, dcf, dsf = oracle.backward(go, x, cf, sf, k, d, s, combine)
        tot = (go * o).sum()
        assert torch.allclose((dx * x).sum(), tot, rtol=1e-10)
        if combine == 'mul':
            assert torch.allclose((dcf * cf).sum(), tot, rtol=1e-10)
            assert torch.allclose((dsf * sf).sum(), tot, rtol=1e-10)
        else:
            assert torch.allclose((dcf * cf).sum() + (dsf * sf).sum(), tot, rtol=1e-10)


@pytest.mark.parametrize('shape', [(1, 70, 10, 10), (35, 1, 10, 10), (1, 1, 50, 50)])
def test_gradcheck_shapes_of_reference(shape):
    """The k=3 shapes of grad_check.py:139-218 through the C oracle against
    autograd (the reference ran torch.autograd.gradcheck on them on a GPU)."""
    N, C, H, W = shape
    for d, s, combine in itertools.product((1, 2), (1, 2), ('mul', 'add')):
        x, cf, sf, go = rand_case(N, C, H, W, 3, s)
        want = oracle.unfold_backward(go, x, cf, sf, 3, d, s, combine)
        got = oracle.backward(go, x, cf, sf, 3, d, s, combine)
        for g, w in zip(got, want):
            assert torch.allclose(g, w, rtol=0, atol=1e-10)


def test_f32_variant_tracks_f64():
    x, cf, sf, go = oracle.make_inputs(2, 8, 14, 14, 3, 1, torch.float32)
    o64 = oracle.forward(x, cf, sf)
    o32 = oracle.forward_f32(x, cf, sf)
    assert o32.dtype == torch.float32
    assert (o32.double() - o64).abs().max() / o64.abs().max() < 1e-6
    g64 = oracle.backward(go, x, cf, sf)
    g32 = oracle.backward_f32(go, x, cf, sf)
    for a, b in zip(g32, g64):
        assert (a.double() - b).abs().max() / b.abs().max() < 1e-6


def test_filter_standardize_closed_form():
    """Unbiased std (divide by n-1) and +1e-10, as ddf/ddf.py:149-150."""
    v = torch.tensor([1., 2., 3., 4., 5., 6., 7., 8., 9.], dtype=torch.float64)
    out = oracle.filter_standardize(v.view(1, 9, 1, 1), 1).view(-1)
    std = (60.0 / 8.0) ** 0.5  # sum (v-5)^2 = 60
    assert torch.allclose(out, (v - 5.0) / (std + 1e-10), atol=1e-14)


def test_make_inputs_is_deterministic_and_standardized():
    a = oracle.make_inputs(2, 4, 14, 14, 3, 1, torch.float32)
    b = oracle.make_inputs(2, 4, 14, 14, 3, 1, torch.float32)
    for u, v in zip(a, b):
        assert torch.equal(u, v)
    _, cf, sf, _ = a
    assert cf.view(2, 4, 9).mean(2).abs().max() < 1e-6
    assert (cf.view(2, 4, 9).std(2) - 1).abs().max() < 1e-5
    assert sf.mean(1).abs().max() < 1e-6
    assert (sf.std(1) - 1).abs().max() < 1e-5


# ---------------------------------------------------------------------------
# committed known-answer fixtures (tests/golden/*.npz, written by
# tests/golden/make_fixtures.py from the loop form and torch autograd)
# ---------------------------------------------------------------------------
def golden_cases():
    import glob
    import os
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')
    return sorted(glob.glob(os.path.join(here, '*.npz')))


def load_golden(path):
    import numpy as np
    z = np.load(path, allow_pickle=False)
    t = {n: torch.from_numpy(z[n]) for n in ('x', 'cf', 'sf', 'go', 'out', 'dx', 'dcf', 'dsf')}
    return t, int(z['k']), int(z['d']), int(z['s']), 'mul' if int(z['combine']) == 0 else 'add'


def test_golden_fixtures_exist():
    assert len(golden_cases()) >= 8


@pytest.mark.parametrize('path', golden_cases(), ids=lambda p: p.split('/')[-1][:-4])
def test_c_oracle_reproduces_golden_fixtures(path):
    """The compiled oracle (the checker of every GPU test) against the frozen
    loop-form / autograd results: fp64 to 1e-12, fp32 entry points to 1e-5."""
    t, k, d, s, combine = load_golden(path)
    out = oracle.forward(t['x'], t['cf'], t['sf'], k, d, s, combine)
    grads = oracle.backward(t['go'], t['x'], t['cf'], t['sf'], k, d, s, combine)
    for got, name in zip((out,) + tuple(grads), ('out', 'dx', 'dcf', 'dsf')):
        scale = max(t[name].abs().max().item(), 1e-30)
        assert (got - t[name]).abs().max().item() / scale < 1e-12, name
    f = [t[n].float() for n in ('x', 'cf', 'sf', 'go')]
    out32 = oracle.forward_f32(f[0], f[1], f[2], k, d, s, combine)
    g32 = oracle.backward_f32(f[3], f[0], f[1], f[2], k, d, s, combine)
    for got, name in zip((out32,) + tuple(g32), ('out', 'dx', 'dcf', 'dsf')):
        scale = max(t[name].abs().max().item(), 1e-30)
        assert (got.double() - t[name]).abs().max().item() / scale < 1e-5, name


# ---------------------------------------------------------------------------
# up-sampling composition (DDFUpPack.forward, ddf/ddf.py:264-272)
# ---------------------------------------------------------------------------
def _up_inputs(N, C, H, W, k, scale, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(N, C, H, W, generator=g, dtype=torch.float64)
    cfs = [torch.randn(N, C, k, k, generator=g, dtype=torch.float64) for _ in range(scale ** 2)]
    sfs = [torch.randn(N, k * k, H, W, generator=g, dtype=torch.float64) for _ in range(scale ** 2)]
    go = torch.randn(N, C, H * scale, W * scale, generator=g, dtype=torch.float64)
    return x, cfs, sfs, go


def _stack_and_shuffle(x, cfs, sfs, k, d, scale, combine):
    """The reference's expression, on the differentiable unfold form."""
    outs = [oracle.unfold_forward(x, cf, sf, k, d, 1, combine) for cf, sf in zip(cfs, sfs)]
    b, c, h, w = outs[0].shape
    return F.pixel_shuffle(torch.stack(outs, dim=2).reshape(b, -1, h, w), scale)


@pytest.mark.parametrize('k,d,scale,combine', [(3, 1, 2, 'mul'), (3, 2, 3, 'add'), (5, 1, 2, 'mul'),
                                               (1, 1, 4, 'add')])
def test_up_forward_is_stack_plus_pixel_shuffle(k, d, scale, combine):
    x, cfs, sfs, _ = _up_inputs(2, 3, 5, 4, k, scale, seed=k + scale)
    got = oracle.up_forward(x, cfs, sfs, k, d, scale, combine)
    want = _stack_and_shuffle(x, cfs, sfs, k, d, scale, combine)
    assert torch.allclose(got, want, atol=1e-12)


def test_up_forward_places_each_branch_on_its_own_lattice():
    """With identity taps and unit spatial filters branch b returns b+1 times
    the features; the result must hold (i*scale + j + 1) * x on lattice (i, j)."""
    x = torch.arange(1., 13.).view(1, 1, 3, 4).double()
    cfs = []
    for b in range(4):
        cf = torch.zeros(1, 1, 3, 3, dtype=torch.float64)
        cf[0, 0, 1, 1] = b + 1
        cfs.append(cf)
    sfs = [torch.ones(1, 9, 3, 4, dtype=torch.float64) for _ in range(4)]
    out = oracle.up_forward(x, cfs, sfs, 3, 1, 2, 'mul')
    for i in range(2):
        for j in range(2):
            assert torch.equal(out[0, 0, i::2, j::2], (i * 2 + j + 1) * x[0, 0])


@pytest.mark.parametrize('k,d,scale,combine', [(3, 1, 2, 'mul'), (3, 2, 2, 'add'), (1, 1, 3, 'mul')])
def test_up_backward_is_autograd_of_the_composition(k, d, scale, combine):
    x, cfs, sfs, go = _up_inputs(2, 3, 4, 5, k, scale, seed=7)
    leaves = [t.clone().requires_grad_(True) for t in [x] + cfs + sfs]
    n = scale ** 2
    out = _stack_and_shuffle(leaves[0], leaves[1:1 + n], leaves[1 + n:], k, d, scale, combine)
    want = torch.autograd.grad(out, leaves, go)
    dx, dcfs, dsfs = oracle.up_backward(go, x, cfs, sfs, k, d, scale, combine)
    assert torch.allclose(dx, want[0], atol=1e-11)
    for b in range(n):
        assert torch.allclose(dcfs[b], want[1 + b], atol=1e-11)
        assert torch.allclose(dsfs[b], want[1 + n + b], atol=1e-11)
