"""Helpers shared by the GPU parity tests."""
import torch

import oracle

# Tolerances on max|got - want| / max|want| against the fp64 oracle evaluated
# on the same (already rounded) inputs.  fp32 and fp16 are the bounds the
# build targets (1e-5 and 1e-2); fp64 is the reference's own forward check
# (grad_check.py:44, 1e-10 absolute on O(1) data) with margin.
TOL = {torch.float64: 1e-12, torch.float32: 1e-5, torch.float16: 1e-2}


def rel_err(got, want):
    want = want.double()
    got = got.detach().double().cpu()
    assert got.shape == want.shape, (got.shape, want.shape)
    if want.numel() == 0:
        return 0.0
    assert torch.isfinite(got).all(), 'non-finite values in result'
    scale = want.abs().max().item()
    return (got - want).abs().max().item() / (scale if scale > 0 else 1.0)


def random_case(N, C, H, W, k, s, dtype, seed=0, standardize=False):
    """CPU tensors (x, cf, sf, go) already rounded to ``dtype``."""
    return oracle.make_inputs(N, C, H, W, k, s, dtype, standardize=standardize, seed=seed)


def to_dev(*ts):
    return tuple(t.cuda() for t in ts)


def run_ddf(x, cf, sf, go, k, d, s, combine, version='', need=(True, True, True)):
    """Forward + backward through the public ``ddf`` autograd function.
    Returns (out, dx, dcf, dsf) with ``None`` for gradients not requested."""
    from ddfnet_amd import ddf
    xd, cfd, sfd, god = to_dev(x, cf, sf, go)
    leaves = [t.requires_grad_(n) for t, n in zip((xd, cfd, sfd), need)]
    out = ddf(leaves[0], leaves[1], leaves[2], k, d, s, combine, version)
    grads = [None, None, None]
    if any(need):
        wanted = [t for t, n in zip(leaves, need) if n]
        got = torch.autograd.grad(out, wanted, god)
        it = iter(got)
        grads = [next(it) if n else None for n in need]
    torch.cuda.synchronize()
    return (out.detach(),) + tuple(grads)


def check_against_oracle(x, cf, sf, go, k, d, s, combine, version='', tol=None, what=''):
    tol = TOL[x.dtype] if tol is None else tol
    out, dx, dcf, dsf = run_ddf(x, cf, sf, go, k, d, s, combine, version)
    assert out.dtype == x.dtype and dx.dtype == x.dtype
    want_o = oracle.forward(x, cf, sf, k, d, s, combine)
    want_g = oracle.backward(go, x, cf, sf, k, d, s, combine)
    errs = {'out': rel_err(out, want_o)}
    for name, g, w in zip(('dX', 'dCF', 'dSF'), (dx, dcf, dsf), want_g):
        errs[name] = rel_err(g, w)
    bad = {n: e for n, e in errs.items() if not e <= tol}
    assert not bad, '%s %s exceeds tol %g: %s' % (what, dict(k=k, d=d, s=s, combine=combine,
                                                              version=version), tol, errs)
    return errs
