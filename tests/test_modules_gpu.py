"""Callers of the operator on the GPU: DDFPack, DDFUpPack and a DDF-ResNet,
against the same modules evaluated on the CPU in fp64 with the oracle standing
in for the HIP operator (same weights, same inputs)."""
import copy

import pytest
import torch

import oracle
import ddfnet_amd
from ddfnet_amd import modules as ddf_modules

pytestmark = pytest.mark.gpu


class _OracleOp(object):
    """``ddf`` replacement for CPU fp64 modules: the differentiable unfold form."""

    def __call__(self, x, cf, sf, k=3, d=1, s=1, combine='mul', version=''):
        return oracle.unfold_forward(x, cf, sf, k, d, s, combine)


def _oracle_up(x, cfs, sfs, k=3, d=1, scale=2, combine='mul'):
    """``ddf_up`` replacement: the reference's composition (ddf/ddf.py:264-272)."""
    outs = [oracle.unfold_forward(x, cf, sf, k, d, 1, combine) for cf, sf in zip(cfs, sfs)]
    b, c, h, w = outs[0].shape
    return torch.nn.functional.pixel_shuffle(torch.stack(outs, dim=2).reshape(b, -1, h, w), scale)


def cpu_reference(module, monkeypatch, *inputs):
    ref = copy.deepcopy(module).cpu().double()
    monkeypatch.setattr(ddf_modules, 'ddf', _OracleOp())
    monkeypatch.setattr(ddf_modules, 'ddf_up', _oracle_up)
    ins = [t.detach().cpu().double().requires_grad_(True) for t in inputs]
    out = ref(*ins)
    monkeypatch.undo()
    return ref, ins, out


@pytest.mark.parametrize('fused', [True, False])
@pytest.mark.parametrize('combine', ['mul', 'add'])
@pytest.mark.parametrize('stride,head', [(1, 1), (2, 1), (1, 4)])
def test_ddfpack_matches_cpu_reference(stride, head, combine, fused, monkeypatch):
    """fused: the spatial filter normalisation and the operator as one autograd node
    (its gradient rides on the operator's partial-sum launch); else op by op."""
    torch.manual_seed(0)
    pack = ddfnet_amd.DDFPack(16, kernel_size=3, stride=stride, head=head,
                              kernel_combine=combine).cuda()
    pack.fuse_spatial_norm = fused
    calls = []
    real = ddf_modules.functional.ddf_spatial_norm
    monkeypatch.setattr(ddf_modules.functional, 'ddf_spatial_norm',
                        lambda *a, **kw: (calls.append(1), real(*a, **kw))[1])
    x = torch.randn(2, 16, 12, 12, device='cuda', requires_grad=True)
    out = pack(x)
    assert calls == ([1] if fused else [])
    assert out.shape == (2, 16, 12 // stride, 12 // stride)
    go = torch.randn_like(out)
    out.backward(go)
    ref, (xr,), out_r = cpu_reference(pack, monkeypatch, x)
    out_r.backward(go.cpu().double())
    assert torch.allclose(out.detach().cpu().double(), out_r.detach(), rtol=1e-4, atol=1e-5)
    assert torch.allclose(x.grad.cpu().double(), xr.grad, rtol=1e-3, atol=1e-4)
    for (name, p), (_, pr) in zip(pack.named_parameters(), ref.named_parameters()):
        assert torch.allclose(p.grad.cpu().double(), pr.grad, rtol=1e-3, atol=1e-4), name


@pytest.mark.parametrize('dtype,tol', [(torch.float32, 2e-4), (torch.float16, 2e-2)])
@pytest.mark.parametrize('k,stride,head,c,hw', [(3, 1, 1, 16, 12), (3, 2, 1, 16, 12), (3, 1, 4, 16, 9),
                                                (5, 1, 1, 70, 10), (3, 1, 1, 300, 7), (3, 1, 2, 64, 30)])
def test_ddfpack_inference_path_matches_cpu_reference(k, stride, head, c, hw, dtype, tol, monkeypatch):
    """Without gradients the two filter branches run as one launch each
    (ddf_hip_channel_branch, ddf_hip_spatial_branch); checked against the CPU
    fp64 modules and against the op-by-op path the same module takes in training."""
    torch.manual_seed(3)
    pack = ddfnet_amd.DDFPack(c, kernel_size=k, stride=stride, head=head).cuda().to(dtype)
    x = torch.randn(3, c, hw, hw + 2, device='cuda').to(dtype)
    with torch.no_grad():
        assert pack._inference_filters(x) is not None       # the one-launch branches do run
        out = pack(x)
        # the ctypes route of the same launches (what runs without the torch extension)
        monkeypatch.setattr(ddf_modules.functional, 'extension', lambda retry=False: None)
        cf, sf = pack._inference_filters(x)
        monkeypatch.undo()
        g = head
        again = ddfnet_amd.ddf(x.reshape(3 * g, c // g, hw, hw + 2), cf.reshape(3 * g, c // g, k, k),
                               sf.reshape(3 * g, k * k, hw // stride, (hw + 2) // stride), k, 1, stride)
        assert torch.equal(out, again.reshape(out.shape))
    _, _, out_r = cpu_reference(pack, monkeypatch, x)
    err = (out.double().cpu() - out_r.detach()).abs().max() / out_r.detach().abs().max()
    assert err < tol, err
    trained = pack(x.clone().requires_grad_(True))           # op-by-op branches
    assert (out.float() - trained.detach().float()).abs().max() / out.float().abs().max() < tol


def test_ddfpack_inference_path_only_for_stock_branches():
    pack = ddfnet_amd.DDFPack(16).cuda()
    x = torch.randn(2, 16, 8, 8, device='cuda')
    with torch.no_grad():
        assert pack._inference_filters(x) is not None
        assert pack._inference_filters(x.double()) is None           # dtype the kernels lack
    assert pack._inference_filters(x) is None                         # parameters want gradients
    with torch.no_grad():
        handle = pack.spatial_branch[0].register_forward_hook(lambda m, i, o: o)
        assert pack._inference_filters(x) is None                     # somebody listens
        handle.remove()
        pack.channel_branch[1] = torch.nn.Conv2d(16, 3, 1, groups=1, padding=1).cuda()
        assert pack._inference_filters(x) is None                     # not a plain 1x1 product
    with torch.no_grad(), torch.autocast('cuda', dtype=torch.float16):
        pack = ddfnet_amd.DDFPack(16).cuda()
        out = pack(x.half())                                          # fp16 features, fp32 parameters
        assert torch.isfinite(out).all()


def test_ddfpack_odd_size_under_stride_fails_in_both_modes():
    """A 1x1 convolution of stride s yields ceil(H / s) rows and the operator
    wants H // s: the reference fails at its reshape (ddf/ddf.py:215-218), with
    and without gradients."""
    pack = ddfnet_amd.DDFPack(16, stride=2).cuda()
    x = torch.randn(2, 16, 9, 8, device='cuda')
    with torch.no_grad():
        assert pack._inference_filters(x) is None
        with pytest.raises(RuntimeError):
            pack(x)
    with pytest.raises(RuntimeError):
        pack(x)


def test_ddfuppack_matches_cpu_reference(monkeypatch):
    torch.manual_seed(1)
    up = ddfnet_amd.DDFUpPack(8, kernel_size=3, scale_factor=2).cuda()
    x = torch.randn(2, 8, 10, 10, device='cuda')
    out = up(x)
    assert out.shape == (2, 8, 20, 20)
    _, _, out_r = cpu_reference(up, monkeypatch, x)
    assert torch.allclose(out.detach().cpu().double(), out_r.detach(), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize('k,scale,head,combine', [(3, 2, 2, 'add'), (3, 3, 1, 'mul'), (5, 2, 1, 'mul'),
                                                  (3, 4, 1, 'mul'), (7, 2, 1, 'mul')])
def test_ddfuppack_trains_like_cpu_reference(k, scale, head, combine, monkeypatch):
    """Forward, input gradient and every parameter gradient of the up-sampling
    pack; (7, 2) has no fused kernel and takes the composed route."""
    torch.manual_seed(3)
    # the guidance convolution pads by kernel_size // 2 (ddf/ddf.py:244-245), so
    # it keeps the plane size only when it is kernel_size wide
    up = ddfnet_amd.DDFUpPack(8, kernel_size=k, scale_factor=scale, head=head,
                              dw_kernel_size=k, kernel_combine=combine).cuda()
    x = torch.randn(2, 8, 9, 7, device='cuda', requires_grad=True)
    out = up(x)
    assert out.shape == (2, 8, 9 * scale, 7 * scale)
    go = torch.randn_like(out)
    out.backward(go)
    ref, (xr,), out_r = cpu_reference(up, monkeypatch, x)
    out_r.backward(go.cpu().double())
    assert torch.allclose(out.detach().cpu().double(), out_r.detach(), rtol=1e-4, atol=1e-5)
    assert torch.allclose(x.grad.cpu().double(), xr.grad, rtol=1e-3, atol=1e-4)
    for (name, p), (_, pr) in zip(up.named_parameters(), ref.named_parameters()):
        assert torch.allclose(p.grad.cpu().double(), pr.grad, rtol=1e-3, atol=1e-4), name


def test_ddfuppack_with_joint_guidance(monkeypatch):
    torch.manual_seed(2)
    up = ddfnet_amd.DDFUpPack(8, kernel_size=3, scale_factor=2, joint_channels=8).cuda()
    x = torch.randn(1, 8, 6, 6, device='cuda')
    joint = torch.randn(1, 8, 6, 6, device='cuda')
    out = up(x, joint)
    _, _, out_r = cpu_reference(up, monkeypatch, x, joint)
    assert torch.allclose(out.detach().cpu().double(), out_r.detach(), rtol=1e-4, atol=1e-5)


def test_ddfpack_fp16_keeps_dtype():
    pack = ddfnet_amd.DDFPack(32).cuda().half()
    x = torch.randn(2, 32, 14, 14, device='cuda', dtype=torch.float16)
    out = pack(x)
    assert out.dtype == torch.float16 and torch.isfinite(out).all()


def test_ddfpack_under_autocast():
    """fp16 activations meet fp32 parameters inside the filter branches; the
    operator promotes its operands to one dtype."""
    pack = ddfnet_amd.DDFPack(32).cuda()
    x = torch.randn(2, 32, 14, 14, device='cuda')
    with torch.autocast('cuda', dtype=torch.float16):
        out = pack(x)
    want = pack(x)
    assert torch.isfinite(out).all()
    assert (out.float() - want).abs().max() / want.abs().max() < 2e-2
    # training step under autocast: gradients reach the input and every parameter
    x.requires_grad_(True)
    with torch.autocast('cuda', dtype=torch.float16):
        loss = pack(x).float().square().mean()
    loss.backward()
    ref = ddfnet_amd.DDFPack(32).cuda()
    ref.load_state_dict(pack.state_dict())
    xr = x.detach().clone().requires_grad_(True)
    ref(xr).square().mean().backward()
    assert (x.grad - xr.grad).abs().max() / xr.grad.abs().max() < 5e-2
    for (name, p_), (_, q) in zip(pack.named_parameters(), ref.named_parameters()):
        assert p_.grad is not None, name
        assert (p_.grad - q.grad).abs().max() / q.grad.abs().max().clamp_min(1e-12) < 5e-2, name


def test_resnet50_forward_matches_cpu_reference(monkeypatch):
    """ddf_mul_resnet50 at a reduced resolution (64x64, batch 2): 16 DDF layers
    at four plane sizes and both strides, fp32 against the CPU fp64 model."""
    from ddfnet_amd import ddf_resnet
    torch.manual_seed(3)
    model = ddf_resnet.ddf_mul_resnet50(num_classes=10, zero_init_last_bn=False).cuda().eval()
    x = torch.randn(2, 3, 64, 64, device='cuda')
    with torch.no_grad():
        out = model(x)
        assert out.shape == (2, 10)
        ref = copy.deepcopy(model).cpu().double()
        monkeypatch.setattr(ddf_modules, 'ddf', _OracleOp())
        out_r = ref(x.cpu().double())
    scale = out_r.abs().max().item()
    assert (out.cpu().double() - out_r).abs().max().item() <= 1e-3 * scale


def test_resnet50_fp16_forward_matches_cpu_reference(monkeypatch):
    """The same network in fp16 on the GPU (the dtype of the batch-128 inference
    configuration; every DDF layer then runs the fp16 kernels) against the CPU
    fp64 model holding the same fp16-rounded weights and input.  Tolerance 2e-2
    of the largest logit: 50+ layers of fp16 activations and BatchNorm, of which
    the DDF layers are held to 1e-2 each at operator level."""
    from ddfnet_amd import ddf_resnet
    torch.manual_seed(5)
    model = ddf_resnet.ddf_mul_resnet50(num_classes=10, zero_init_last_bn=False).cuda().half().eval()
    x = torch.randn(2, 3, 64, 64, device='cuda').half()
    with torch.no_grad():
        out = model(x)
        assert out.dtype == torch.float16 and out.shape == (2, 10)
        ref = copy.deepcopy(model).cpu().double()
        monkeypatch.setattr(ddf_modules, 'ddf', _OracleOp())
        out_r = ref(x.cpu().double())
    assert torch.isfinite(out).all()
    scale = out_r.abs().max().item()
    assert (out.cpu().double() - out_r).abs().max().item() <= 2e-2 * scale


def test_resnet50_fp16_inference_and_layer_timing():
    from ddfnet_amd import ddf_resnet
    torch.manual_seed(4)
    model = ddf_resnet.ddf_mul_resnet50(zero_init_last_bn=False).cuda().half().eval()
    x = torch.randn(4, 3, 224, 224, device='cuda', dtype=torch.float16)
    with torch.no_grad():
        out = model(x)
    assert out.shape == (4, 1000) and torch.isfinite(out).all()
    layers = ddf_resnet.time_ddf_layers(model, x, iters=2)
    shapes = [(l['shape'][1], l['shape'][2], l['stride']) for l in layers]
    # the 16 DDF call shapes of ResNet-50 at 224x224
    want = ([(64, 56, 1)] * 3 + [(128, 56, 2)] + [(128, 28, 1)] * 3 + [(256, 28, 2)] +
            [(256, 14, 1)] * 5 + [(512, 14, 2)] + [(512, 7, 1)] * 2)
    assert shapes == want


def test_resnet50_with_folded_batchnorm_computes_the_same_function():
    """fold_batchnorm folds the eval-mode BatchNorms that follow convolutions into
    them: same logits (fp32, non-trivial running statistics), fewer modules."""
    from ddfnet_amd import ddf_resnet
    torch.manual_seed(5)
    model = ddf_resnet.ddf_mul_resnet50(num_classes=10, zero_init_last_bn=False).cuda()
    for m in model.modules():
        if isinstance(m, torch.nn.BatchNorm2d):
            torch.nn.init.uniform_(m.weight, 0.5, 1.5)
            torch.nn.init.uniform_(m.bias, -0.2, 0.2)
            m.running_mean.uniform_(-0.1, 0.1)
            m.running_var.uniform_(0.5, 1.5)
    model.eval()
    folded = ddf_resnet.fold_batchnorm(model)
    n_bn = lambda net: sum(isinstance(m, torch.nn.BatchNorm2d) for m in net.modules())
    assert n_bn(model) == 53 and n_bn(folded) == 16   # one per block remains (after the DDF layer)
    x = torch.randn(2, 3, 64, 64, device='cuda')
    with torch.no_grad():
        want, got = model(x), folded(x)
    assert (got - want).abs().max().item() <= 1e-4 * want.abs().max().item()
    with pytest.raises(AssertionError):
        ddf_resnet.fold_batchnorm(model.train())


# ---------------------------------------------------------------------------
# fused filter normalisation
# ---------------------------------------------------------------------------
@pytest.mark.parametrize('dtype,tol', [(torch.float64, 1e-12), (torch.float32, 1e-5),
                                       (torch.float16, 1e-2)])
@pytest.mark.parametrize('ftype,shape,groups,k,rstd,rmean', [
    ('spatial', (3, 9, 13, 11), 1, 3, False, False),
    ('spatial', (2, 4 * 9, 7, 5), 4, 3, True, True),
    ('spatial', (1, 25, 6, 6), 1, 5, False, True),
    ('channel', (4, 16 * 9), 16, 3, True, False),
    ('channel', (2, 5 * 25, 1, 1), 5, 5, True, True),
    ('channel', (3, 7 * 9), 7, 3, False, False),
])
def test_fused_filter_norm_matches_formula(ftype, shape, groups, k, rstd, rmean, dtype, tol):
    """One HIP launch against the op-by-op formulation of the same module
    evaluated in fp64 on the CPU."""
    torch.manual_seed(3)
    fn = ddfnet_amd.FilterNorm(groups, k, ftype, 'relu', running_std=rstd,
                               running_mean=rmean).cuda().to(dtype)
    x = (torch.randn(*shape) * 2 + 0.5).to(dtype).cuda()
    with torch.no_grad():
        assert fn._use_fused(x)
        got = fn(x)
    assert got.dtype == dtype
    ref = copy.deepcopy(fn).cpu().double()
    want = ref(x.detach().cpu().double())
    assert got.shape == want.shape
    err = (got.cpu().double() - want.detach()).abs().max().item() / want.abs().max().item()
    assert err <= tol, err


@pytest.mark.parametrize('dtype,tol', [(torch.float64, 1e-11), (torch.float32, 2e-5),
                                       (torch.float16, 1e-2)])
@pytest.mark.parametrize('ftype,shape,groups,k,rstd,rmean', [
    ('spatial', (3, 9, 13, 11), 1, 3, False, False),
    ('spatial', (2, 4 * 9, 7, 5), 4, 3, True, True),
    ('spatial', (1, 25, 6, 6), 1, 5, False, True),
    ('channel', (4, 16 * 9), 16, 3, True, False),
    ('channel', (2, 5 * 25, 1, 1), 5, 5, True, True),
    ('channel', (3, 7 * 9), 7, 3, False, False),
])
def test_fused_filter_norm_gradients(ftype, shape, groups, k, rstd, rmean, dtype, tol):
    """The one-launch backward against torch.autograd through the op-by-op
    formulation of the same module in fp64 on the CPU: gradient of the input,
    of the learned gain and of the learned offset."""
    torch.manual_seed(4)
    fn = ddfnet_amd.FilterNorm(groups, k, ftype, 'relu', running_std=rstd,
                               running_mean=rmean).cuda().to(dtype)
    x = (torch.randn(*shape) * 2 + 0.5).to(dtype).cuda().requires_grad_(True)
    assert fn._use_fused(x)
    out = fn(x)
    go = torch.randn(out.shape).to(dtype).cuda()
    out.backward(go)
    ref = copy.deepcopy(fn).cpu().double()
    ref.zero_grad()
    xr = x.detach().cpu().double().requires_grad_(True)
    ref(xr).backward(go.cpu().double())

    def err(got, want):
        return (got.cpu().double() - want).abs().max().item() / want.abs().max().item()

    assert err(x.grad, xr.grad) <= tol
    if rstd:
        assert err(fn.std.grad, ref.std.grad) <= tol
    if rmean:
        assert err(fn.mean.grad, ref.mean.grad) <= tol


def test_filter_norm_gradient_only_where_asked():
    fn = ddfnet_amd.FilterNorm(8, 3, 'channel', 'relu', running_std=True).cuda()
    fn.std.requires_grad_(False)
    x = torch.randn(2, 72, device='cuda', requires_grad=True)
    fn(x).sum().backward()
    assert x.grad is not None and fn.std.grad is None
    x2 = torch.randn(2, 72, device='cuda')
    fn.std.requires_grad_(True)
    fn(x2).sum().backward()
    assert fn.std.grad is not None


def test_filter_norm_cpu_path_is_op_by_op():
    fn = ddfnet_amd.FilterNorm(2, 3, 'spatial')
    x = torch.randn(1, 18, 4, 4, requires_grad=True)
    assert not fn._use_fused(x)
    fn(x).sum().backward()
    assert x.grad is not None
