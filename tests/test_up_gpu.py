"""The fused up-sampling operator (``ddf_up`` / ``ddf_hip_up_forward``) against
the oracle's composition of per-branch forwards and a pixel shuffle."""
import ctypes

import pytest
import torch

import oracle
import ddfnet_amd
from ddfnet_amd import _lib, ddf, ddf_up
from ddf_testlib import TOL, rel_err

pytestmark = pytest.mark.gpu


def up_case(N, C, H, W, k, scale, dtype, seed=0):
    """CPU tensors already rounded to ``dtype``: x, [cf_b], [sf_b], go."""
    g = torch.Generator(device='cpu').manual_seed(seed)
    base = torch.float64 if dtype == torch.float64 else torch.float32
    x = torch.randn(N, C, H, W, generator=g, dtype=base).to(dtype)
    cfs = [torch.randn(N, C, k, k, generator=g, dtype=base).to(dtype) for _ in range(scale ** 2)]
    sfs = [torch.randn(N, k * k, H, W, generator=g, dtype=base).to(dtype)
           for _ in range(scale ** 2)]
    go = torch.randn(N, C, H * scale, W * scale, generator=g, dtype=base).to(dtype)
    return x, cfs, sfs, go


def check_up(N, C, H, W, k, d, scale, combine, dtype, backward=True, seed=0):
    x, cfs, sfs, go = up_case(N, C, H, W, k, scale, dtype, seed)
    xd = x.cuda().requires_grad_(backward)
    cfd = [t.cuda().requires_grad_(backward) for t in cfs]
    sfd = [t.cuda().requires_grad_(backward) for t in sfs]
    out = ddf_up(xd, cfd, sfd, k, d, scale, combine)
    assert out.dtype == dtype and out.shape == (N, C, H * scale, W * scale)
    tol = TOL[dtype]
    errs = {'out': rel_err(out, oracle.up_forward(x, cfs, sfs, k, d, scale, combine))}
    if backward:
        grads = torch.autograd.grad(out, [xd] + cfd + sfd, go.cuda())
        want_x, want_cf, want_sf = oracle.up_backward(go, x, cfs, sfs, k, d, scale, combine)
        errs['dX'] = rel_err(grads[0], want_x)
        for b in range(scale ** 2):
            errs['dCF%d' % b] = rel_err(grads[1 + b], want_cf[b])
            errs['dSF%d' % b] = rel_err(grads[1 + scale ** 2 + b], want_sf[b])
    bad = {n: e for n, e in errs.items() if not e <= tol}
    assert not bad, (dict(N=N, C=C, H=H, W=W, k=k, d=d, scale=scale, combine=combine), errs)


@pytest.mark.parametrize('dtype', [torch.float64, torch.float32, torch.float16])
@pytest.mark.parametrize('combine', ['mul', 'add'])
@pytest.mark.parametrize('k,scale', [(1, 2), (1, 3), (1, 4), (3, 2), (3, 3), (3, 4), (5, 2)])
def test_every_fused_kernel(k, scale, combine, dtype):
    """Odd plane (not a multiple of the block), odd channel count."""
    check_up(2, 5, 9, 13, k, 1, scale, combine, dtype)


@pytest.mark.parametrize('d', [2, 3])
@pytest.mark.parametrize('k,scale', [(3, 2), (5, 2), (3, 3)])
def test_dilation(k, scale, d):
    check_up(1, 4, 11, 10, k, d, scale, 'mul', torch.float32)


@pytest.mark.parametrize('N,C,H,W', [
    (1, 70, 40, 36),    # channels split over blocks and staged in two rounds
    (3, 33, 17, 16),    # last chunk shorter than the others
    (1, 1, 1, 1), (1, 2, 1, 300), (1, 2, 300, 1),
    (4, 8, 16, 16),     # block count a multiple of 8: renumbered across XCDs
    (1, 200, 8, 8),     # many stages in one block
])
def test_shapes(N, C, H, W):
    check_up(N, C, H, W, 3, 1, 2, 'mul', torch.float32)


def test_empty_tensors():
    for shape in ((0, 4, 5, 5), (2, 0, 5, 5), (2, 4, 0, 5)):
        N, C, H, W = shape
        x = torch.zeros(shape, device='cuda')
        cfs = [torch.zeros(N, C, 3, 3, device='cuda') for _ in range(4)]
        sfs = [torch.zeros(N, 9, H, W, device='cuda') for _ in range(4)]
        assert ddf_up(x, cfs, sfs, 3, 1, 2).shape == (N, C, 2 * H, 2 * W)


def test_unsupported_pair_composes_from_ddf():
    """(k, scale) = (7, 2) and (5, 3) have no fused kernel."""
    lib = _lib.lib()
    x = torch.zeros(1, 1, 4, 4, device='cuda')
    ptrs = (ctypes.c_void_p * 16)(*([x.data_ptr()] * 16))
    rc = lib.ddf_hip_up_forward(x.data_ptr(), ptrs, ptrs, x.data_ptr(), 1, 1, 4, 4, 7, 1, 2, 0, 1,
                                None)
    assert rc == 2 and b'does not cover' in lib.ddf_hip_last_error()
    check_up(2, 6, 10, 9, 7, 1, 2, 'mul', torch.float32)
    check_up(1, 4, 8, 9, 5, 1, 3, 'add', torch.float32)


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16])
@pytest.mark.parametrize('scale', [2, 4])
def test_misaligned_output(scale, dtype):
    """A result that starts one element past an aligned address cannot take
    one aligned store per row."""
    x, cfs, sfs, _ = up_case(2, 6, 7, 9, 3, scale, dtype, seed=5)
    xd, cfd, sfd = x.cuda(), [t.cuda() for t in cfs], [t.cuda() for t in sfs]
    n = 2 * 6 * 7 * 9 * scale * scale
    buf = torch.full((n + 2,), 7.0, device='cuda', dtype=dtype)
    out = buf[1:1 + n].view(2, 6, 7 * scale, 9 * scale)
    assert out.data_ptr() % (2 * out.element_size()) == out.element_size()
    _lib.up_forward(xd, cfd, sfd, out, 3, 1, scale, 'mul')
    torch.cuda.synchronize()
    assert rel_err(out, oracle.up_forward(x, cfs, sfs, 3, 1, scale, 'mul')) <= TOL[dtype]
    assert buf[0].item() == 7.0 and buf[-1].item() == 7.0    # nothing outside the result


def test_backward_routes_agree():
    """The gradient runs all branches as one batch on the row-register kernels;
    features that are not 16-byte aligned take the branch-by-branch route."""
    x, cfs, sfs, go = up_case(2, 6, 8, 12, 3, 2, torch.float32, seed=9)
    want_x, want_cf, want_sf = oracle.up_backward(go, x, cfs, sfs, 3, 1, 2, 'mul')
    cfd, sfd, god = [t.cuda() for t in cfs], [t.cuda() for t in sfs], go.cuda()
    buf = torch.zeros(x.numel() + 1, device='cuda')
    for shift in (0, 1):
        xd = buf[shift:shift + x.numel()].view_as(x)
        xd.copy_(x)
        assert xd.data_ptr() % 16 == 4 * shift
        gx = torch.empty(x.shape, device='cuda')
        gcf = [torch.empty_like(t) for t in cfd]
        gsf = [torch.empty_like(t) if b != 2 else None for b, t in enumerate(sfd)]   # one not wanted
        _lib.up_backward(god, xd, cfd, sfd, gx, gcf, gsf, 3, 1, 2, 'mul')
        torch.cuda.synchronize()
        assert rel_err(gx, want_x) <= 1e-5
        for b in range(4):
            assert rel_err(gcf[b], want_cf[b]) <= 1e-5
            if gsf[b] is not None:
                assert rel_err(gsf[b], want_sf[b]) <= 1e-5


def test_mixed_dtypes_and_partial_gradients():
    """fp16 features with fp32 filters promote to fp32; only the gradients
    asked for come back."""
    x, cfs, sfs, go = up_case(1, 4, 6, 6, 3, 2, torch.float32, seed=2)
    xd = x.half().cuda()
    cfd = [t.cuda() for t in cfs]
    sfd = [t.cuda().requires_grad_(b == 1) for b, t in enumerate(sfs)]
    out = ddf_up(xd, cfd, sfd, 3, 1, 2, 'mul')
    assert out.dtype == torch.float32
    (g,) = torch.autograd.grad(out, [sfd[1]], go.cuda())
    _, _, want_sf = oracle.up_backward(go, x.half().float(), cfs, sfs, 3, 1, 2, 'mul')
    assert rel_err(g, want_sf[1]) <= 1e-5


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16])
def test_full_size_equals_composition_of_ddf(dtype):
    """At a size the CPU oracle would take long for: the fused launch against
    ``ddf`` per branch + ``pixel_shuffle`` (kernels that the parity tests of the
    operator cover), and linearity in the features."""
    N, C, H, W, k, scale = 4, 64, 96, 96, 3, 2
    g = torch.Generator(device='cuda').manual_seed(0)
    x = torch.randn(N, C, H, W, device='cuda', generator=g).to(dtype)
    cfs = [torch.randn(N, C, k, k, device='cuda', generator=g).to(dtype) / 3 for _ in range(4)]
    sfs = [torch.randn(N, k * k, H, W, device='cuda', generator=g).to(dtype) for _ in range(4)]
    out = ddf_up(x, cfs, sfs, k, 1, scale, 'mul')
    outs = [ddf(x, cf, sf, k, 1, 1, 'mul') for cf, sf in zip(cfs, sfs)]
    want = torch.nn.functional.pixel_shuffle(torch.stack(outs, 2).reshape(N, -1, H, W), scale)
    tol = 1e-5 if dtype == torch.float32 else 2e-3
    assert rel_err(out, want.cpu()) <= tol
    if dtype == torch.float32:
        x2 = torch.randn(N, C, H, W, device='cuda', generator=g)
        both = ddf_up(x + 2 * x2, cfs, sfs, k, 1, scale, 'mul')
        assert rel_err(both, (out + 2 * ddf_up(x2, cfs, sfs, k, 1, scale, 'mul')).cpu()) <= 1e-5


def test_ddfuppack_uses_the_fused_operator(monkeypatch):
    from ddfnet_amd import functional
    up = ddfnet_amd.DDFUpPack(8, scale_factor=2).cuda()
    x = torch.randn(1, 8, 6, 6, device='cuda')

    def no_branch_calls(*a, **kw):
        raise AssertionError('the per-branch composition ran')
    monkeypatch.setattr(functional, 'ddf', no_branch_calls)
    with torch.no_grad():
        out = up(x)                      # C++ operator where the torch extension is built
    # the ctypes route of the same library call
    calls = []
    real = _lib.up_forward
    monkeypatch.setattr(functional, 'extension', lambda retry=False: None)
    monkeypatch.setattr(_lib, 'up_forward', lambda *a: (calls.append(1), real(*a))[1])
    with torch.no_grad():
        again = up(x)
    assert calls == [1] and torch.equal(out, again)


def _random_up_cases(count, seed):
    import random
    rng = random.Random(seed)
    for _ in range(count):
        k, scale = rng.choice([(1, 2), (1, 3), (1, 4), (3, 2), (3, 2), (3, 3), (3, 4), (5, 2), (7, 2)])
        yield (rng.randint(1, 3), rng.randint(1, 40), rng.randint(1, 23), rng.randint(1, 23), k,
               rng.choice([1, 1, 2, 3]), scale, rng.choice(['mul', 'add']),
               rng.choice([torch.float64, torch.float32, torch.float16]))


@pytest.mark.parametrize('chunk', range(3))
def test_random_shapes_against_oracle(chunk):
    """60 seeded random problems, forward and every gradient."""
    for i, (N, C, H, W, k, d, scale, combine, dtype) in enumerate(_random_up_cases(20, 500 + chunk)):
        check_up(N, C, H, W, k, d, scale, combine, dtype, seed=chunk * 100 + i)


def test_up_forward_replays_in_a_hip_graph():
    """The fused launch enqueues one kernel and allocates only its result, so
    it can be captured; every replay, with eager work in between, reproduces
    the eager result bit for bit."""
    N, C, H, W, k, scale = 2, 24, 12, 10, 3, 2
    cases = [up_case(N, C, H, W, k, scale, torch.float32, seed=s) for s in (31, 32, 33)]
    x = cases[0][0].cuda()
    cfs = [t.cuda() for t in cases[0][1]]
    sfs = [t.cuda() for t in cases[0][2]]

    def step():
        with torch.no_grad():
            return ddf_up(x, cfs, sfs, k, 1, scale, 'mul')

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for cx, ccfs, csfs, _ in cases:
        x.copy_(cx.cuda())
        for dst, src in zip(cfs + sfs, ccfs + csfs):
            dst.copy_(src.cuda())
        graph.replay()
        torch.cuda.synchronize()
        got = captured.clone()
        want = step()
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        assert rel_err(got, oracle.up_forward(cx, ccfs, csfs, k, 1, scale, 'mul')) <= 1e-5
