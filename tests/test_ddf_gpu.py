"""GPU parity tests: the HIP kernels, reached through the public ``ddf``
function and the C ABI, against the CPU oracle on identical seeded inputs.

Tolerances (see ddf_testlib.TOL): fp64 1e-12, fp32 1e-5, fp16 1e-2 on
max|got-want| / max|want|.  Shapes follow the reference's own test script
(grad_check.py:33-299) and extend it with the edge cases it leaves out."""
import ctypes
import itertools

import pytest
import torch

import oracle
from ddf_testlib import (TOL, check_against_oracle, random_case, rel_err, run_ddf, to_dev)

pytestmark = pytest.mark.gpu

DTYPES = [torch.float64, torch.float32, torch.float16]
VERSIONS = ['', 'o']


def _ids(v):
    return str(v).replace('torch.', '')


# ---------------------------------------------------------------------------
# shapes of the reference's test script
# ---------------------------------------------------------------------------
@pytest.mark.parametrize('version', ['o', 'f', ''])
@pytest.mark.parametrize('d', [1, 2])
def test_reference_forward_check(d, version):
    """grad_check.py:33-73: 1x10x15x15 fp64, k=3, 'mul', versions 'o' and 'f'
    against the loop form; the reference's bound is 1e-10 absolute."""
    g = torch.Generator().manual_seed(3)
    x = torch.randn(1, 10, 15, 15, generator=g, dtype=torch.float64)
    cf = torch.randn(1, 10, 3, 3, generator=g, dtype=torch.float64)
    sf = torch.randn(1, 9, 15, 15, generator=g, dtype=torch.float64)
    want = oracle.loop_forward(x, cf, sf, 3, d, 1, 'mul')
    from ddfnet_amd import ddf
    got = ddf(x.cuda(), cf.cuda(), sf.cuda(), 3, d, 1, 'mul', version).cpu()
    assert (got - want).abs().max().item() <= 1e-10


@pytest.mark.parametrize('shape', [(96, 64, 56, 56), (96, 128, 28, 28), (96, 256, 14, 14),
                                   (96, 512, 7, 7)], ids=_ids)
def test_reference_o_equals_f(shape):
    """grad_check.py:77-133: version 'o' and 'f' agree to 1e-10 in fp64 at the
    four ResNet stage shapes (batch 96)."""
    from ddfnet_amd import ddf
    N, C, H, W = shape
    g = torch.Generator(device='cuda').manual_seed(5)
    x = torch.randn(N, C, H, W, generator=g, dtype=torch.float64, device='cuda')
    cf = torch.randn(N, C, 3, 3, generator=g, dtype=torch.float64, device='cuda')
    sf = torch.randn(N, 9, H, W, generator=g, dtype=torch.float64, device='cuda')
    o = ddf(x, cf, sf, 3, 1, 1, 'mul', 'o')
    f = ddf(x, cf, sf, 3, 1, 1, 'mul', 'f')
    assert (o - f).abs().max().item() <= 1e-10


GRADCHECK_SHAPES = {3: [(1, 70, 10, 10), (35, 1, 10, 10), (1, 1, 50, 50)],
                    5: [(1, 70, 10, 10), (20, 1, 10, 10), (1, 1, 40, 40)]}


@pytest.mark.parametrize('version', VERSIONS)
@pytest.mark.parametrize('dtype', DTYPES, ids=_ids)
@pytest.mark.parametrize('k', [3, 5])
def test_reference_gradcheck_shapes_vs_oracle(k, dtype, version):
    """grad_check.py:139-299: 3 shapes x d in {1,2} x s in {1,2} x {mul,add}
    per kernel size.  The reference differentiated numerically on the GPU; here
    every output and gradient is compared with the oracle, whose gradients are
    themselves pinned by numerical differentiation on the CPU."""
    for (N, C, H, W), d, s, combine in itertools.product(
            GRADCHECK_SHAPES[k], (1, 2), (1, 2), ('mul', 'add')):
        case = random_case(N, C, H, W, k, s, dtype, seed=N + C + H)
        check_against_oracle(*case, k, d, s, combine, version, what=str((N, C, H, W)))


@pytest.mark.parametrize('combine', ['mul', 'add'])
@pytest.mark.parametrize('k,d,s', [(3, 1, 1), (3, 2, 2), (5, 1, 2)])
def test_numerical_gradcheck_small(k, d, s, combine):
    """torch.autograd.gradcheck on the device with the reference's settings
    (atol=1e-5, eps=1e-3; grad_check.py:144)."""
    from ddfnet_amd import ddf
    x, cf, sf, _ = random_case(2, 3, 8, 6, k, s, torch.float64, seed=11)
    x, cf, sf = (t.cuda().requires_grad_(True) for t in (x, cf, sf))
    assert torch.autograd.gradcheck(ddf, (x, cf, sf, k, d, s, combine), atol=1e-5, eps=1e-3)


@pytest.mark.parametrize('combine', ['mul', 'add'])
def test_config1_gradcheck_scale(combine):
    """N=2, C=16, 14x14 fp64, k=3 d=1 s=1: outputs and all three gradients
    against the oracle, then a fast-mode numerical gradcheck."""
    from ddfnet_amd import ddf
    case = random_case(2, 16, 14, 14, 3, 1, torch.float64, seed=0)
    check_against_oracle(*case, 3, 1, 1, combine)
    x, cf, sf = (t.cuda().requires_grad_(True) for t in case[:3])
    assert torch.autograd.gradcheck(ddf, (x, cf, sf, 3, 1, 1, combine), atol=1e-5, eps=1e-3,
                                    fast_mode=True)


# ---------------------------------------------------------------------------
# edge cases the reference's script leaves out
# ---------------------------------------------------------------------------
EDGE = [
    # N, C, H, W, k, d, s
    (2, 3, 9, 11, 3, 1, 2),     # odd sizes with stride 2: floor(H/s)
    (1, 5, 2, 2, 3, 1, 1),      # image smaller than the window
    (1, 5, 3, 4, 5, 2, 1),      # dilated window far larger than the image
    (2, 4, 7, 7, 1, 1, 1),      # k = 1
    (2, 4, 9, 9, 1, 1, 2),      # k = 1, strided
    (1, 6, 12, 12, 7, 1, 1),    # k = 7
    (1, 3, 13, 13, 3, 3, 3),    # dilation and stride 3
    (3, 65, 14, 14, 3, 1, 1),   # C one past a wavefront
    (2, 130, 7, 7, 3, 1, 1),    # 7x7 plane, C not a multiple of 64
    (1, 2, 1, 1, 3, 1, 1),      # single pixel
    (1, 1, 1, 64, 3, 1, 1),     # single row
    (1, 1, 64, 1, 3, 1, 1),     # single column
    (2, 3, 20, 30, 3, 1, 1),    # W not a multiple of anything nice
    (1, 2, 5, 200, 5, 1, 2),    # wide and short
    (1, 2, 31, 17, 3, 2, 1),    # primes
    (1, 8, 3, 3, 3, 1, 4),      # stride larger than the window: Ho=Wo=0
    (1, 4, 20, 300, 3, 1, 1),   # wide: several lane segments per row
    (2, 8, 33, 224, 3, 1, 2),   # wide, strided, odd height
    (1, 2, 5, 513, 5, 1, 1),    # wider than the tuned kernels' 8 x 64 columns
    (1, 3, 130, 6, 3, 2, 1),    # tall and narrow
    (1, 3, 113, 128, 3, 1, 1),  # large plane: two rows per lane, odd height
    (1, 2, 60, 264, 3, 1, 1),   # large plane, rows of two segments, two rows per lane
    (1, 2, 48, 264, 5, 2, 1),   # 5x5 dilated on segmented rows
    (2, 2, 9, 1000, 3, 1, 1),   # five segments per row
]


@pytest.mark.parametrize('combine', ['mul', 'add'])
@pytest.mark.parametrize('case', [(1, 2, 50, 272, 3, 1, 1), (1, 3, 57, 520, 3, 1, 1), (2, 2, 16, 264, 5, 1, 1),
                                  (1, 4, 31, 304, 3, 2, 1)], ids=_ids)
def test_wide_rows_fp16(case, combine):
    """fp16 rows of more than 32 eight-pixel vectors are cut into segments."""
    N, C, H, W, k, d, s = case
    tensors = random_case(N, C, H, W, k, s, torch.float16, seed=11)
    check_against_oracle(*tensors, k, d, s, combine, '', what=str(case))


STRIDE2 = [
    # N, C, H, W: 3x3, stride 2
    (2, 10, 56, 56),    # four result pixels per lane (fp32), eight (fp16); four strips per plane
    (2, 7, 28, 28),     # two / four result pixels per lane
    (3, 9, 14, 14),     # 7 x 7 results: one pixel per lane (fp32)
    (1, 5, 33, 64),     # odd height: the last feature row is never read
    (2, 6, 15, 36),     # rows of 18 results, odd height
    (1, 4, 40, 256),    # 32 lanes per result row: no idle lane between rows
    (1, 3, 9, 250),     # result rows longer than a wave's lanes: the tile kernels
    (2, 70, 12, 24),    # more channels than one wave walks
]


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16], ids=_ids)
@pytest.mark.parametrize('combine', ['mul', 'add'])
@pytest.mark.parametrize('shape', STRIDE2, ids=_ids)
def test_stride_two_on_the_row_kernels(shape, combine, dtype):
    """Stride 2: forward and filter gradients run on the row-register kernels
    where a result row fits the lanes of a wave and the feature rows keep their
    vectors aligned; everything against the oracle."""
    from ddfnet_amd import _lib
    N, C, H, W = shape
    if shape in ((2, 10, 56, 56), (2, 7, 28, 28)):
        assert 'k_rows<' in _lib.describe(shape, 3, 1, 2, combine, dtype) and \
            'stride 2' in _lib.describe(shape, 3, 1, 2, combine, dtype)
        assert 'k_rows_filters<' in _lib.describe(shape, 3, 1, 2, combine, dtype, need=7)
    tensors = random_case(N, C, H, W, 3, 2, dtype, seed=13)
    check_against_oracle(*tensors, 3, 1, 2, combine, '', what=str(shape))
    # all gradients together come from one launch where the height is even; asked for
    # separately, the feature gradient is the tile kernel's: the routes agree to rounding
    x, cf, sf, go = tensors
    together = run_ddf(x, cf, sf, go, 3, 1, 2, combine)
    only_dx = run_ddf(x, cf, sf, go, 3, 1, 2, combine, need=(True, False, False))
    only_filters = run_ddf(x, cf, sf, go, 3, 1, 2, combine, need=(False, True, True))
    tol = 1e-6 if dtype == torch.float32 else 2e-3
    assert rel_err(only_dx[1], together[1].cpu()) <= tol
    assert rel_err(only_filters[2], together[2].cpu()) <= tol
    assert rel_err(only_filters[3], together[3].cpu()) <= tol


@pytest.mark.parametrize('version', VERSIONS)
@pytest.mark.parametrize('dtype', [torch.float64, torch.float32], ids=_ids)
@pytest.mark.parametrize('case', EDGE, ids=_ids)
def test_edge_cases(case, dtype, version):
    N, C, H, W, k, d, s = case
    for combine in ('mul', 'add'):
        tensors = random_case(N, C, H, W, k, s, dtype, seed=7)
        check_against_oracle(*tensors, k, d, s, combine, version, what=str(case))


def test_empty_batch_and_channels():
    from ddfnet_amd import ddf
    for N, C in ((0, 4), (2, 0)):
        x = torch.zeros(N, C, 8, 8, device='cuda', requires_grad=True)
        cf = torch.zeros(N, C, 3, 3, device='cuda', requires_grad=True)
        sf = torch.zeros(N, 9, 8, 8, device='cuda', requires_grad=True)
        out = ddf(x, cf, sf, 3, 1, 1, 'mul')
        assert out.shape == (N, C, 8, 8)
        out.sum().backward()
        assert x.grad.shape == x.shape and cf.grad.shape == cf.shape
        assert sf.grad.shape == sf.shape
        if sf.grad.numel():
            assert (sf.grad == 0).all()


# ---------------------------------------------------------------------------
# benchmark configurations at full size
# ---------------------------------------------------------------------------
FULL = {
    'C2': (64, 256, 14, 14, 3, 1, 1, 'mul', torch.float32),
    'C3': (64, 64, 56, 56, 3, 1, 1, 'add', torch.float16),
    'C4a': (32, 128, 56, 56, 3, 1, 2, 'mul', torch.float32),
    'C4b': (32, 128, 56, 56, 5, 2, 1, 'mul', torch.float32),
}


@pytest.mark.parametrize('version', VERSIONS)
@pytest.mark.parametrize('name', sorted(FULL))
def test_full_size_configs(name, version):
    """Standardised filters, seed 0, as the benchmark draws them."""
    N, C, H, W, k, d, s, combine, dtype = FULL[name]
    case = random_case(N, C, H, W, k, s, dtype, seed=0, standardize=True)
    errs = check_against_oracle(*case, k, d, s, combine, version, what=name)
    print(name, version, errs)


# The seven distinct DDF call shapes of ddf_mul_resnet50 (channels, input size, stride):
# three per stage of 56 / 28 / 14 / 7 pixels, the first of stages 2-4 with stride 2.
RESNET50_LAYERS = [(64, 56, 1), (128, 56, 2), (128, 28, 1), (256, 28, 2), (256, 14, 1),
                   (512, 14, 2), (512, 7, 1)]


@pytest.mark.parametrize('dtype', [torch.float16, torch.float32])
@pytest.mark.parametrize('C,size,s', RESNET50_LAYERS)
def test_resnet50_layer_shapes(C, size, s, dtype):
    """'mul', 3 x 3, batch 8, in the precision the network runs in (fp16) and in fp32."""
    case = random_case(8, C, size, size, 3, s, dtype, seed=21, standardize=True)
    check_against_oracle(*case, 3, 1, s, 'mul', what='resnet50 layer C=%d %dx%d s=%d' % (C, size, size, s))


@pytest.mark.parametrize('name', sorted(FULL))
def test_full_size_invariants(name):
    """Size-independent properties on the device results alone.  mul is
    trilinear: <dX,X> = <dCF,CF> = <dSF,SF> = <dO,O>; add: <dX,X> = <dO,O> and
    <dCF,CF> + <dSF,SF> = <dO,O>."""
    N, C, H, W, k, d, s, combine, dtype = FULL[name]
    x, cf, sf, go = random_case(N, C, H, W, k, s, dtype, seed=1, standardize=True)
    out, dx, dcf, dsf = run_ddf(x, cf, sf, go, k, d, s, combine)
    dot = lambda a, b: (a.double().cpu() * b.double().cpu()).sum().item()
    tot = dot(go, out)
    tol = 2e-2 if dtype == torch.float16 else 1e-4
    scale = (go.double().abs() * out.double().cpu().abs()).sum().item()
    assert abs(dot(dx, x) - tot) <= tol * scale
    if combine == 'mul':
        assert abs(dot(dcf, cf) - tot) <= tol * scale
        assert abs(dot(dsf, sf) - tot) <= tol * scale
    else:
        assert abs(dot(dcf, cf) + dot(dsf, sf) - tot) <= tol * scale


def test_closed_form_depthwise_conv_on_device():
    """mul with SF == 1 is a per-sample depthwise convolution (reference
    README.md:49-63), here against torch's own conv2d on the device."""
    import torch.nn.functional as F
    from ddfnet_amd import ddf
    N, C, H, W, k = 4, 32, 28, 28, 3
    g = torch.Generator().manual_seed(2)
    x = torch.randn(N, C, H, W, generator=g).cuda()
    cf = torch.randn(N, C, k, k, generator=g).cuda()
    sf = torch.ones(N, k * k, H, W).cuda()
    got = ddf(x, cf, sf, k, 1, 1, 'mul')
    want = F.conv2d(x.view(1, N * C, H, W).double(), cf.view(N * C, 1, k, k).double(),
                    padding=1, groups=N * C).view(N, C, H, W)
    assert rel_err(got, want.cpu()) <= 1e-5


# ---------------------------------------------------------------------------
# committed known-answer fixtures
# ---------------------------------------------------------------------------
def _golden_paths():
    import glob
    import os
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')
    return sorted(glob.glob(os.path.join(here, '*.npz')))


@pytest.mark.parametrize('version', VERSIONS)
@pytest.mark.parametrize('dtype', DTYPES, ids=_ids)
@pytest.mark.parametrize('path', _golden_paths(), ids=lambda p: p.split('/')[-1][:-4])
def test_golden_fixtures(path, dtype, version):
    """HIP kernels against tests/golden/*.npz (inputs and fp64 results frozen by
    tests/golden/make_fixtures.py).  For fp32 and fp16 the inputs are rounded
    first, so the expected values are recomputed from the rounded inputs by the
    oracle, which test_oracle.py holds to the same fixtures."""
    import numpy as np
    z = np.load(path, allow_pickle=False)
    k, d, s = int(z['k']), int(z['d']), int(z['s'])
    combine = 'mul' if int(z['combine']) == 0 else 'add'
    x, cf, sf, go = (torch.from_numpy(z[n]).to(dtype) for n in ('x', 'cf', 'sf', 'go'))
    got = run_ddf(x, cf, sf, go, k, d, s, combine, version)
    if dtype == torch.float64:
        want = [torch.from_numpy(z[n]) for n in ('out', 'dx', 'dcf', 'dsf')]
    else:
        want = [oracle.forward(x, cf, sf, k, d, s, combine)] + \
            list(oracle.backward(go, x, cf, sf, k, d, s, combine))
    for g, w, name in zip(got, want, ('out', 'dX', 'dCF', 'dSF')):
        assert rel_err(g, w) <= TOL[dtype], name


# ---------------------------------------------------------------------------
# API behaviour
# ---------------------------------------------------------------------------
def test_needs_input_grad_subsets():
    x, cf, sf, go = random_case(2, 6, 10, 10, 3, 1, torch.float32, seed=4)
    full = run_ddf(x, cf, sf, go, 3, 1, 1, 'mul')
    for need in itertools.product((False, True), repeat=3):
        if not any(need):
            continue
        part = run_ddf(x, cf, sf, go, 3, 1, 1, 'mul', need=need)
        for g_full, g_part, n in zip(full[1:], part[1:], need):
            if n:
                # a subset may run other kernels than the full backward (other
                # summation order): equal to rounding, not bit for bit
                assert rel_err(g_part, g_full.cpu()) <= 1e-6
            else:
                assert g_part is None


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16], ids=_ids)
@pytest.mark.parametrize('combine', ['mul', 'add'])
@pytest.mark.parametrize('shape', [(2, 24, 56, 56), (3, 20, 28, 28), (2, 9, 14, 14), (2, 6, 10, 6),
                                   (1, 5, 8, 64), (2, 7, 32, 16), (1, 3, 2, 2), (2, 4, 12, 128)])
def test_stride2_feature_gradient_alone(shape, combine, dtype):
    """dX asked for on its own with stride 2 (what autograd does when the filters are
    frozen): even heights run on the row-register kernel, which writes feature rows 2y
    and 2y + 1 from the lane of result row y."""
    from ddfnet_amd import _lib
    N, C, H, W = shape
    x, cf, sf, go = random_case(N, C, H, W, 3, 2, dtype, seed=17)
    assert 'k_rows<dX' in _lib.describe(shape, 3, 1, 2, combine, dtype, _lib.NEED_DX)
    _, dx, dcf, dsf = run_ddf(x, cf, sf, go, 3, 1, 2, combine, need=(True, False, False))
    assert dcf is None and dsf is None
    want = oracle.backward(go, x, cf, sf, 3, 1, 2, combine)[0]
    assert rel_err(dx, want) <= TOL[dtype]


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16], ids=_ids)
@pytest.mark.parametrize('combine', ['mul', 'add'])
@pytest.mark.parametrize('shape,d', [((3, 40, 14, 14), 1), ((2, 24, 14, 14), 2), ((2, 9, 12, 16), 1),
                                     ((1, 130, 8, 8), 1), ((2, 20, 28, 28), 1), ((2, 12, 56, 56), 1)])
def test_one_launch_backward_equals_separate_requests(shape, d, combine, dtype):
    """All three gradients requested together may come from one fused kernel
    (3x3, stride 1, short strips); requested one at a time - what autograd does
    when only some inputs need gradients - the feature gradient and the filter
    gradients come from kernels of their own.  The routes may order their sums
    differently: they must agree to rounding, and both must match the oracle."""
    N, C, H, W = shape
    x, cf, sf, go = random_case(N, C, H, W, 3, 1, dtype, seed=11)
    together = run_ddf(x, cf, sf, go, 3, d, 1, combine)
    only_dx = run_ddf(x, cf, sf, go, 3, d, 1, combine, need=(True, False, False))
    only_filters = run_ddf(x, cf, sf, go, 3, d, 1, combine, need=(False, True, True))
    tol = 1e-6 if dtype == torch.float32 else 2e-3
    assert rel_err(only_dx[0], together[0].cpu()) == 0.0
    assert rel_err(only_dx[1], together[1].cpu()) <= tol
    assert rel_err(only_filters[2], together[2].cpu()) <= tol
    assert rel_err(only_filters[3], together[3].cpu()) <= tol
    want = oracle.backward(go, x, cf, sf, 3, d, 1, combine)
    for got, w in zip(together[1:], want):
        assert rel_err(got, w) <= TOL[dtype]


def test_mixed_dtypes_are_promoted():
    """fp16 features with fp32 filters: the reference widens the fp16 operand
    (ddf/ddf.py:37-42); result is fp32."""
    from ddfnet_amd import ddf
    x, cf, sf, _ = random_case(2, 4, 8, 8, 3, 1, torch.float32, seed=9)
    got = ddf(x.half().cuda(), cf.cuda(), sf.cuda(), 3, 1, 1, 'mul')
    assert got.dtype == torch.float32
    want = oracle.forward(x.half(), cf, sf, 3, 1, 1, 'mul')
    assert rel_err(got, want) <= 1e-5
    # ... and gradients flow back to every operand in that operand's own dtype
    xh = x.half().cuda().requires_grad_(True)
    cfd, sfd = cf.cuda().requires_grad_(True), sf.cuda().requires_grad_(True)
    out = ddf(xh, cfd, sfd, 3, 1, 1, 'mul')
    go = torch.randn_like(out)
    dx, dcf, dsf = torch.autograd.grad(out, (xh, cfd, sfd), go)
    assert dx.dtype == torch.float16 and dcf.dtype == torch.float32 and dsf.dtype == torch.float32
    wx, wcf, wsf = oracle.backward(go.cpu(), x.half(), cf, sf, 3, 1, 1, 'mul')
    assert rel_err(dx, wx) <= 1e-2 and rel_err(dcf, wcf) <= 1e-5 and rel_err(dsf, wsf) <= 1e-5


def test_non_contiguous_inputs_are_accepted():
    from ddfnet_amd import ddf
    x, cf, sf, _ = random_case(2, 4, 8, 10, 3, 1, torch.float32, seed=10)
    xt = x.cuda().transpose(2, 3).contiguous().transpose(2, 3)  # same values, strided
    assert not xt.is_contiguous()
    got = ddf(xt, cf.cuda(), sf.cuda(), 3, 1, 1, 'add')
    assert rel_err(got, oracle.forward(x, cf, sf, 3, 1, 1, 'add')) <= 1e-5
    # channels_last features and gradients (what a channels_last network hands over)
    xc = x.cuda().to(memory_format=torch.channels_last).requires_grad_(True)
    assert not xc.is_contiguous()
    out = ddf(xc, cf.cuda(), sf.cuda(), 3, 1, 1, 'mul')
    go = torch.randn_like(out).to(memory_format=torch.channels_last)
    (dx,) = torch.autograd.grad(out, xc, go)
    want = oracle.backward(go.cpu().contiguous(), x, cf, sf, 3, 1, 1, 'mul')[0]
    assert out.is_contiguous() and rel_err(dx, want) <= 1e-5


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16], ids=_ids)
@pytest.mark.parametrize('shape,stride', [((2, 16, 14, 14), 1), ((1, 33, 28, 56), 2), ((2, 3, 7, 7), 1),
                                          ((1, 16, 8, 28), 2)])
def test_tensors_that_start_at_odd_addresses(shape, stride, dtype):
    """Contiguous tensors whose first element is one to three elements into an
    allocation (views): the vector kernels turn such pointers down and the call
    falls back to kernels with narrower accesses; results as always."""
    from ddfnet_amd import ddf

    def shifted(t, off):
        base = torch.empty(t.numel() + 8, dtype=t.dtype, device='cuda')
        view = base[off:off + t.numel()].view(t.shape)
        view.copy_(t)
        return view

    for combine, offs in (('mul', (1, 0, 0, 0)), ('add', (0, 0, 1, 2)), ('mul', (3, 1, 2, 1))):
        x, cf, sf, go = random_case(*shape, 3, stride, dtype, seed=sum(offs))
        xd, cfd, sfd, god = (shifted(t.cuda(), o) for t, o in zip((x, cf, sf, go), offs))
        leaves = [t.requires_grad_(True) for t in (xd, cfd, sfd)]
        out = ddf(*leaves, 3, 1, stride, combine)
        grads = torch.autograd.grad(out, leaves, god)
        want = (oracle.forward(x, cf, sf, 3, 1, stride, combine),) + tuple(
            oracle.backward(go, x, cf, sf, 3, 1, stride, combine))
        for got, w in zip((out,) + tuple(grads), want):
            assert rel_err(got.detach(), w) <= TOL[dtype]


def test_runs_on_the_current_stream():
    from ddfnet_amd import ddf
    x, cf, sf, _ = random_case(4, 16, 14, 14, 3, 1, torch.float32, seed=12)
    want = oracle.forward(x, cf, sf, 3, 1, 1, 'mul')
    side = torch.cuda.Stream()
    xd, cfd, sfd = to_dev(x, cf, sf)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        got = ddf(xd, cfd, sfd, 3, 1, 1, 'mul')
    side.synchronize()
    assert rel_err(got, want) <= 1e-5


def test_argument_errors():
    from ddfnet_amd import ddf, OP_DICT
    x, cf, sf, _ = to_dev(*random_case(1, 2, 6, 6, 3, 1, torch.float32))
    with pytest.raises(AssertionError, match='input feature must be a CUDA tensor'):
        ddf(x.cpu(), cf, sf, 3, 1, 1, 'mul')
    with pytest.raises(AssertionError, match='does not match kernel size'):
        ddf(x, cf, sf, 5, 1, 1, 'mul')
    with pytest.raises(AssertionError, match='does not match feature size'):
        ddf(x, cf[:, :1], sf, 3, 1, 1, 'mul')
    with pytest.raises(AssertionError, match='with stride 2'):
        ddf(x, cf, sf, 3, 1, 2, 'mul')
    with pytest.raises(AssertionError, match='only support mul or add'):
        ddf(x, cf, sf, 3, 1, 1, 'max')
    with pytest.raises(RuntimeError, match='must be contiguous'):
        OP_DICT['mul'].forward(x.transpose(2, 3), cf, sf, 3, 1, 1, torch.empty_like(x))
    with pytest.raises(RuntimeError, match='not implemented on CPU'):
        OP_DICT['mul'].forward(x.cpu(), cf, sf, 3, 1, 1, torch.empty_like(x))
    assert OP_DICT['mul_faster'].backward is None


def test_c_abi_directly():
    """Raw ctypes calls with device pointers: status codes and the forward
    result, without the autograd wrapper."""
    from ddfnet_amd import _lib
    lib = _lib.lib()
    x, cf, sf, go = random_case(2, 8, 14, 14, 3, 1, torch.float32, seed=13)
    xd, cfd, sfd, god = to_dev(x, cf, sf, go)
    out = torch.empty_like(xd)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.ddf_hip_forward(p(xd), p(cfd), p(sfd), p(out), 2, 8, 14, 14, 3, 1, 1, 0, 1, 0, stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert rel_err(out, oracle.forward(x, cf, sf)) <= 1e-5
    # even kernel size -> DDF_ERR_BAD_ARG with a message
    rc = lib.ddf_hip_forward(p(xd), p(cfd), p(sfd), p(out), 2, 8, 14, 14, 4, 1, 1, 0, 1, 0, stream)
    assert rc == 1 and b'kernel_size' in lib.ddf_hip_last_error()
    # null pointer
    rc = lib.ddf_hip_forward(None, p(cfd), p(sfd), p(out), 2, 8, 14, 14, 3, 1, 1, 0, 1, 0, stream)
    assert rc == 1
    # backward with workspace handling
    need = 7
    nbytes = lib.ddf_hip_backward_workspace_bytes(2, 8, 14, 14, 3, 1, 1, 0, 1, need, 0)
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device='cuda')
    dx, dcf, dsf = torch.empty_like(xd), torch.empty_like(cfd), torch.empty_like(sfd)
    rc = lib.ddf_hip_backward(p(god), p(xd), p(cfd), p(sfd), p(dx), p(dcf), p(dsf), p(ws), nbytes,
                              2, 8, 14, 14, 3, 1, 1, 0, 1, need, 0, stream)
    assert rc == 0, lib.ddf_hip_last_error()
    torch.cuda.synchronize()
    for g, w in zip((dx, dcf, dsf), oracle.backward(go, x, cf, sf)):
        assert rel_err(g, w) <= 1e-5
    if nbytes:
        rc = lib.ddf_hip_backward(p(god), p(xd), p(cfd), p(sfd), p(dx), p(dcf), p(dsf), None, 0,
                                  2, 8, 14, 14, 3, 1, 1, 0, 1, need, 0, stream)
        assert rc == 3


def test_results_are_deterministic():
    x, cf, sf, go = random_case(8, 64, 14, 14, 3, 1, torch.float32, seed=14, standardize=True)
    a = run_ddf(x, cf, sf, go, 3, 1, 1, 'mul')
    b = run_ddf(x, cf, sf, go, 3, 1, 1, 'mul')
    for u, v in zip(a, b):
        assert torch.equal(u, v)


@pytest.mark.parametrize('shape,stride,dtype', [
    ((4, 32, 14, 14), 1, torch.float32),    # one-launch backward + one partial sum
    ((2, 40, 56, 56), 2, torch.float32),    # stride 2: one-launch backward + both partial sums
    ((3, 20, 7, 7), 1, torch.float16),      # two-byte vectors
], ids=_ids)
def test_forward_and_backward_replay_in_a_hip_graph(shape, stride, dtype):
    """The operator allocates nothing the capture cannot own and enqueues only
    kernels (no memset nodes), so forward + backward can be captured once and
    replayed.  Every replay - with ordinary eager work and synchronisation in
    between - must reproduce the eager result bit for bit."""
    from ddfnet_amd import ddf
    host = [random_case(*shape, 3, stride, dtype, seed=s) for s in (21, 22, 23)]
    x, cf, sf, go = (t.clone().requires_grad_(i < 3) for i, t in enumerate(to_dev(*host[0])))

    def step():
        out = ddf(x, cf, sf, 3, 1, stride, 'mul')
        return (out,) + torch.autograd.grad(out, (x, cf, sf), go)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for case in host:
        with torch.no_grad():
            for dst, src in zip((x, cf, sf, go), to_dev(*case)):
                dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = step()          # eager, between replays
        torch.cuda.synchronize()
        for g, w in zip(got, want):
            assert torch.equal(g, w)


# ---------------------------------------------------------------------------
# seeded random sweep over shapes and parameters
# ---------------------------------------------------------------------------
def _random_cases(count, seed):
    import random
    rng = random.Random(seed)
    cases = []
    while len(cases) < count:
        k = rng.choice([1, 3, 3, 3, 5, 5, 7])
        d = rng.choice([1, 1, 2, 3])
        s = rng.choice([1, 1, 2, 3])
        N, C = rng.randint(1, 4), rng.choice([1, 2, 3, 5, 8, 17, 33, 64, 70])
        H, W = rng.randint(1, 40), rng.randint(1, 70)
        if rng.random() < 0.3:          # the vector paths want friendly row lengths
            W = rng.choice([8, 12, 16, 28, 32, 56, 64])
        combine = rng.choice(['mul', 'add'])
        dtype = rng.choice([torch.float32, torch.float32, torch.float16, torch.float64])
        cases.append((N, C, H, W, k, d, s, combine, dtype))
    return cases


@pytest.mark.parametrize('chunk', range(6))
def test_random_shapes_against_oracle(chunk):
    """120 seeded random problems (all kernel families, ragged sizes, empty
    outputs when the stride exceeds the image) through the default variant."""
    for i, (N, C, H, W, k, d, s, combine, dtype) in enumerate(_random_cases(20, 1000 + chunk)):
        case = random_case(N, C, H, W, k, s, dtype, seed=chunk * 100 + i)
        check_against_oracle(*case, k, d, s, combine, '',
                             what='chunk %d case %d %s' % (chunk, i, (N, C, H, W, str(dtype))))


@pytest.mark.parametrize('chunk', range(3))
def test_random_stride_two_and_odd_rows_against_oracle(chunk):
    """Seeded random 3x3 problems aimed at the stride-2 row kernels (all vector
    widths, odd heights, rows too long for them) and at fp16 rows of odd length."""
    import random
    rng = random.Random(4000 + chunk)
    done = 0
    while done < 40:
        s = rng.choice([1, 2, 2])
        dtype = rng.choice([torch.float16, torch.float32, torch.float16])
        N, C = rng.randint(1, 3), rng.choice([1, 2, 3, 7, 16, 33, 64, 65, 130])
        H = rng.randint(1, 40)
        W = rng.choice([1, 2, 3, 4, 6, 7, 8, 10, 12, 14, 15, 16, 20, 24, 28, 30, 32, 36, 48, 56, 57, 64, 66,
                        128, 130, 256, 258])
        if H // s == 0 or W // s == 0:
            continue
        combine = rng.choice(['mul', 'add'])
        case = random_case(N, C, H, W, 3, s, dtype, seed=chunk * 1000 + done)
        check_against_oracle(*case, 3, 1, s, combine, '',
                             what=str((N, C, H, W, s, combine, dtype)))
        done += 1


def test_tensors_beyond_2_31_elements():
    """66 x 512 x 256 x 256 fp16 is 2.2e9 elements: offsets no longer fit 32
    bits (the reference indexes with int, ddf_mul_cuda_kernel.cu:28-33).  The
    last sample, which lies wholly beyond 2^31, must come out exactly as when
    it is run on its own, forward and all gradients."""
    from ddfnet_amd import ddf
    free, _ = torch.cuda.mem_get_info()
    if free < 40 * 2 ** 30:
        pytest.skip('needs about 40 GiB of device memory')
    N, C, H, W = 66, 512, 256, 256
    g = torch.Generator(device='cuda').manual_seed(77)
    x = torch.randn(N, C, H, W, generator=g, device='cuda', dtype=torch.float16)
    cf = torch.randn(N, C, 3, 3, generator=g, device='cuda', dtype=torch.float16)
    sf = torch.randn(N, 9, H, W, generator=g, device='cuda', dtype=torch.float16)
    assert x.numel() > 2 ** 31
    x.requires_grad_(True); cf.requires_grad_(True); sf.requires_grad_(True)
    out = ddf(x, cf, sf, 3, 1, 1, 'mul')
    go = torch.randn(N, C, H, W, generator=g, device='cuda', dtype=torch.float16)
    dx, dcf, dsf = torch.autograd.grad(out, (x, cf, sf), go)
    n = N - 1
    xs, cfs, sfs = (t[n:].detach().clone().requires_grad_(True) for t in (x, cf, sf))
    outs = ddf(xs, cfs, sfs, 3, 1, 1, 'mul')
    dxs, dcfs, dsfs = torch.autograd.grad(outs, (xs, cfs, sfs), go[n:].clone())
    assert torch.equal(out[n:], outs) and torch.equal(dx[n:], dxs)
    assert torch.equal(dcf[n:], dcfs) and torch.equal(dsf[n:], dsfs)
    # and the single sample against the oracle (a few channels of it)
    sl = slice(0, 4)
    want = oracle.forward(xs[:, sl].detach().cpu(), cfs[:, sl].detach().cpu(), sfs.detach().cpu(),
                          3, 1, 1, 'mul')
    assert rel_err(outs[:, sl], want) <= TOL[torch.float16]


@pytest.mark.parametrize('dtype', [torch.float64, torch.float32, torch.float16])
@pytest.mark.parametrize('N,C,H,W,d,combine', [
    (3, 37, 7, 7, 1, 'mul'),     # 5 channel planes per workgroup pass, ragged channel count
    (2, 130, 7, 7, 2, 'add'),    # taps staged in two rounds
    (1, 3, 8, 8, 1, 'mul'),      # fewer channels than plane slots
    (2, 19, 3, 20, 2, 'mul'), (2, 19, 20, 3, 1, 'add'),
    (1, 300, 1, 1, 1, 'mul'), (2, 9, 1, 64, 1, 'mul'), (4, 64, 4, 4, 1, 'mul'),
])
def test_tiny_planes(N, C, H, W, d, combine, dtype):
    """Planes of at most 64 pixels take the kernels that pack several channel
    planes into one workgroup pass (forward and feature gradient)."""
    case = random_case(N, C, H, W, 3, 1, dtype, seed=N + C)
    check_against_oracle(*case, 3, d, 1, combine, '', what='tiny plane')
    check_against_oracle(*case, 3, d, 1, combine, 'f', what='tiny plane, tiled forced')


@pytest.mark.parametrize('combine', ['mul', 'add'])
@pytest.mark.parametrize('N,C,H,W,s', [
    (3, 37, 7, 7, 1), (2, 20, 15, 15, 1), (1, 9, 6, 31, 1), (2, 6, 33, 57, 1),   # odd row lengths
    (3, 20, 14, 14, 2), (2, 9, 12, 30, 2), (1, 5, 11, 14, 2),                     # odd result rows
])
def test_fp16_rows_of_odd_length(N, C, H, W, s, combine):
    """fp16 rows with an odd number of pixels: one pixel (two bytes) per lane on the
    row-register kernels."""
    from ddfnet_amd import _lib
    assert 'k_rows<VX=1' in _lib.describe((N, C, H, W), 3, 1, s, combine, torch.float16)
    assert 'k_rows_filters<' in _lib.describe((N, C, H, W), 3, 1, s, combine, torch.float16, need=7)
    case = random_case(N, C, H, W, 3, s, torch.float16, seed=N + C + W)
    check_against_oracle(*case, 3, 1, s, combine, '', what='fp16, odd rows')
    x, cf, sf, go = case
    together = run_ddf(x, cf, sf, go, 3, 1, s, combine)
    only_dx = run_ddf(x, cf, sf, go, 3, 1, s, combine, need=(True, False, False))
    only_filters = run_ddf(x, cf, sf, go, 3, 1, s, combine, need=(False, True, True))
    assert rel_err(only_dx[1], together[1].cpu()) <= 2e-3
    assert rel_err(only_filters[2], together[2].cpu()) <= 2e-3
    assert rel_err(only_filters[3], together[3].cpu()) <= 2e-3


def test_cpp_operator_equals_python_operator():
    """ddf is the C++ autograd function of the torch extension where that is
    built; DDFFunction is the Python one.  Same checks, same library calls:
    results and gradients are bit-identical."""
    from ddfnet_amd import DDFFunction, ddf, functional
    if functional.extension() is None:
        pytest.skip('torch extension not built')
    for dtype in (torch.float32, torch.float16):
        for (N, C, H, W, k, d, s, combine) in [(2, 16, 14, 14, 3, 1, 1, 'mul'), (2, 8, 9, 11, 3, 2, 2, 'add'),
                                               (1, 4, 12, 12, 5, 1, 1, 'mul')]:
            x, cf, sf, go = oracle.make_inputs(N, C, H, W, k, s, dtype)
            a = [t.cuda().requires_grad_(True) for t in (x, cf, sf)]
            b = [t.cuda().requires_grad_(True) for t in (x, cf, sf)]
            out_a = ddf(*a, k, d, s, combine)
            out_b = DDFFunction.apply(*b, k, d, s, combine)
            assert torch.equal(out_a, out_b)
            ga = torch.autograd.grad(out_a, a, go.cuda())
            gb = torch.autograd.grad(out_b, b, go.cuda())
            for u, v in zip(ga, gb):
                assert torch.equal(u, v)
    # mixed dtypes are promoted, only the wanted gradients are computed
    x, cf, sf, go = oracle.make_inputs(2, 8, 10, 10, 3, 1, torch.float32)
    xh = x.cuda().half().requires_grad_(True)
    out = ddf(xh, cf.cuda(), sf.cuda())
    assert out.dtype == torch.float32
    (gx,) = torch.autograd.grad(out, [xh], go.cuda())
    assert gx.dtype == torch.float16 and gx.shape == xh.shape
    # keyword arguments and defaults as in the reference's signature
    assert torch.equal(ddf(x.cuda(), cf.cuda(), sf.cuda(), kernel_combine='add', kernel_size=3),
                       DDFFunction.apply(x.cuda(), cf.cuda(), sf.cuda(), 3, 1, 1, 'add'))
    with torch.autocast('cuda', dtype=torch.float16):
        assert ddf(x.cuda(), cf.cuda(), sf.cuda()).dtype == torch.float16
