"""The one-launch filter branches of DDFPack through the C ABI
(ddf_hip_spatial_branch, ddf_hip_channel_branch) against fp64 restatements of
the reference modules they replace: the 1x1 convolution with the operator's
stride followed by FilterNorm('spatial') (ddf/ddf.py:176-180, :145-157), and
the bottleneck MLP on the pooled features followed by FilterNorm('channel')
(ddf/ddf.py:183-192, :158-170)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from ddfnet_amd import _lib  # noqa: E402


def spatial_reference(x, w, b, head, k, s, gain, gain_vec, offset_vec):
    kk = k * k
    n, c, h, wd = x.shape
    ho, wo = h // s, wd // s
    xs = x.double()[:, :, :ho * s:s, :wo * s:s]
    u = torch.einsum('oc,nchw->nohw', w.double().view(head * kk, c), xs)
    if b is not None:
        u = u + b.double().view(1, -1, 1, 1)
    u = u.view(n, head, kk, ho, wo)
    m = u.mean(2, keepdim=True)
    r = (u - m) / ((u - m).std(2, keepdim=True) + 1e-10)
    r = r * (gain if gain_vec is None else gain_vec.double().view(1, head, kk, 1, 1))
    if offset_vec is not None:
        r = r + offset_vec.double().view(1, head, kk, 1, 1)
    return r.view(n, head * kk, ho, wo)


def channel_reference(pooled, w1, b1, w2, b2, k, gain, gain_vec, offset_vec):
    kk = k * k
    n, c = pooled.shape
    hdn = torch.relu(pooled.double() @ w1.double().t() + b1.double())
    u = (hdn @ w2.double().t() + b2.double()).view(n, c, kk)
    m = u.mean(2, keepdim=True)
    r = (u - m) / ((u - m).std(2, keepdim=True) + 1e-10)
    r = r * (gain if gain_vec is None else gain_vec.double().view(1, c, kk))
    if offset_vec is not None:
        r = r + offset_vec.double().view(1, c, kk)
    return r.view(n, c, k, k)


# (N, C, H, W, stride, head): the ResNet-50 layer shapes at a small batch, planes
# whose size rules out one vector width after the other, odd sizes under stride 2,
# several heads, channel counts that are no multiple of the kernel's channel group
SPATIAL_CASES = [
    (3, 16, 12, 14, 1, 1), (3, 16, 12, 14, 2, 1), (3, 16, 9, 11, 1, 4), (2, 300, 7, 7, 1, 1),
    (3, 64, 30, 32, 1, 2), (2, 64, 56, 56, 1, 1), (2, 128, 56, 56, 2, 1), (2, 128, 28, 28, 1, 1),
    (2, 256, 28, 28, 2, 1), (2, 256, 14, 14, 1, 1), (2, 512, 14, 14, 2, 1), (2, 512, 7, 7, 1, 1),
    (1, 8, 5, 3, 1, 1), (1, 6, 5, 3, 2, 1), (2, 36, 13, 17, 2, 3), (1, 4, 64, 64, 1, 1),
    (5, 1024, 7, 9, 1, 1), (2, 20, 40, 24, 2, 2), (2, 7, 10, 12, 1, 1), (40, 32, 28, 28, 1, 1),
]


@pytest.mark.parametrize('dtype,tol', [(torch.float32, 2e-5), (torch.float16, 4e-3)])
@pytest.mark.parametrize('case', SPATIAL_CASES, ids=lambda c: 'x'.join(map(str, c)))
@pytest.mark.parametrize('vectors', [False, True])
def test_spatial_branch_matches_fp64(case, vectors, dtype, tol):
    n, c, h, w_, s, head = case
    torch.manual_seed(hash(case) % 1000)
    x = torch.randn(n, c, h, w_, device='cuda').to(dtype)
    w = (torch.randn(head * 9, c, device='cuda') * 0.2).to(dtype)
    b = torch.randn(head * 9, device='cuda').to(dtype) if vectors else None
    gv = (torch.rand(head * 9, device='cuda') + 0.5).to(dtype) if vectors else None
    ov = torch.randn(head * 9, device='cuda').to(dtype) if vectors else None
    out = _lib.spatial_branch(x, w, b, head, 3, s, 0.7, gv, ov)
    ref = spatial_reference(*(None if t is None else t.cpu() for t in (x, w, b)), head, 3, s, 0.7,
                            None if gv is None else gv.cpu(), None if ov is None else ov.cpu())
    assert out.shape == ref.shape
    err = ((out.double().cpu() - ref).abs().max() / ref.abs().max()).item()
    assert err < tol, err


@pytest.mark.parametrize('dtype,tol', [(torch.float32, 2e-5), (torch.float16, 4e-3)])
def test_spatial_branch_unaligned_views(dtype, tol):
    """Tensors that start at odd element offsets: the vector widths fall back."""
    torch.manual_seed(5)
    for shift in (1, 2, 3):
        n, c, h, w_ = 2, 24, 12, 16
        store = torch.randn(n * c * h * w_ + shift, device='cuda').to(dtype)
        x = store[shift:].view(n, c, h, w_)
        w = (torch.randn(9, c, device='cuda') * 0.2).to(dtype)
        out = _lib.spatial_branch(x, w, None, 1, 3, 1, 1.0, None, None)
        ref = spatial_reference(x.cpu(), w.cpu(), None, 1, 3, 1, 1.0, None, None)
        err = ((out.double().cpu() - ref).abs().max() / ref.abs().max()).item()
        assert err < tol, (shift, err)


@pytest.mark.parametrize('dtype,tol', [(torch.float32, 2e-5), (torch.float16, 6e-3)])
@pytest.mark.parametrize('n,c,k', [(3, 16, 3), (128, 64, 3), (5, 128, 3), (4, 256, 3), (3, 512, 3),
                                   (2, 70, 5), (7, 300, 3), (2, 1024, 3), (3, 64, 5), (6, 96, 3),
                                   (130, 512, 3), (9, 256, 5),
                                   # fp16 on the matrix cores: hidden layers of exactly one step, of a
                                   # step and a few values, of several steps; batches that end inside a tile
                                   (16, 160, 3), (4, 192, 3), (20, 320, 3), (2, 448, 5), (33, 1024, 3),
                                   (17, 1280, 3)])
def test_channel_branch_matches_fp64(n, c, k, dtype, tol):
    torch.manual_seed(n + c)
    mid = int(c * 0.2)
    pooled = torch.randn(n, c, device='cuda').to(dtype)
    w1 = (torch.randn(mid, c, device='cuda') * 0.2).to(dtype)
    b1 = torch.randn(mid, device='cuda').to(dtype)
    w2 = (torch.randn(c * k * k, mid, device='cuda') * 0.3).to(dtype)
    b2 = torch.randn(c * k * k, device='cuda').to(dtype)
    gv = (torch.rand(c * k * k, device='cuda') + 0.5).to(dtype)
    ov = torch.randn(c * k * k, device='cuda').to(dtype)
    out = _lib.channel_branch(pooled, w1, b1, w2, b2, k, 1.0, gv, ov)
    ref = channel_reference(*(t.cpu() for t in (pooled, w1, b1, w2, b2)), k, 1.0, gv.cpu(), ov.cpu())
    err = ((out.double().cpu() - ref).abs().max() / ref.abs().max()).item()
    assert err < tol, err


@pytest.mark.parametrize('n,c,k', [(5, 256, 3), (18, 512, 3), (3, 160, 5), (4, 64, 3)])
def test_channel_branch_without_biases_and_vectors(n, c, k):
    """Scalar gain, no offset, no biases (fp16: the matrix-core kernel where the shape allows it)."""
    torch.manual_seed(c)
    mid = int(c * 0.2)
    pooled = torch.randn(n, c, device='cuda').half()
    w1 = (torch.randn(mid, c, device='cuda') * 0.2).half()
    w2 = (torch.randn(c * k * k, mid, device='cuda') * 0.3).half()
    out = _lib.channel_branch(pooled, w1, None, w2, None, k, 0.7, None, None)
    zeros1, zeros2 = torch.zeros(mid), torch.zeros(c * k * k)
    ref = channel_reference(pooled.cpu(), w1.cpu(), zeros1, w2.cpu(), zeros2, k, 0.7, None, None)
    err = ((out.double().cpu() - ref).abs().max() / ref.abs().max()).item()
    assert err < 6e-3, err


def test_channel_branch_operands_at_odd_addresses():
    """Weights, biases and vectors that start 2 bytes into their allocations (views of
    larger tensors): whichever kernel takes the call, the taps are the same as from
    aligned copies."""
    torch.manual_seed(3)
    n, c, k = 20, 256, 3
    mid = int(c * 0.2)

    def shifted(t):
        store = torch.empty(t.numel() + 1, device='cuda', dtype=t.dtype)
        view = store[1:].view(t.shape)
        view.copy_(t)
        return view

    pooled = torch.randn(n, c, device='cuda').half()
    w1 = (torch.randn(mid, c, device='cuda') * 0.2).half()
    b1 = torch.randn(mid, device='cuda').half()
    w2 = (torch.randn(c * k * k, mid, device='cuda') * 0.3).half()
    b2 = torch.randn(c * k * k, device='cuda').half()
    gv = (torch.rand(c * k * k, device='cuda') + 0.5).half()
    ov = torch.randn(c * k * k, device='cuda').half()
    want = _lib.channel_branch(pooled, w1, b1, w2, b2, k, 1.0, gv, ov)
    ref = channel_reference(*(t.cpu() for t in (pooled, w1, b1, w2, b2)), k, 1.0, gv.cpu(), ov.cpu())
    scale = ref.abs().max()
    for which in range(7):
        args = [pooled, w1, b1, w2, b2, gv, ov]
        args[which] = shifted(args[which])
        out = _lib.channel_branch(args[0], args[1], args[2], args[3], args[4], k, 1.0, args[5], args[6])
        assert ((out.double().cpu() - ref).abs().max() / scale).item() < 6e-3, which
        assert ((out.float() - want.float()).abs().max() / scale).item() < 2e-3, which


POOL_CASES = [(2, 64, 56, 56, 1, 1), (2, 128, 56, 56, 2, 1), (2, 128, 28, 28, 1, 1), (2, 256, 28, 28, 2, 1),
              (2, 256, 14, 14, 1, 1), (2, 512, 14, 14, 2, 1), (2, 512, 7, 7, 1, 1), (3, 16, 12, 14, 1, 1),
              (3, 16, 12, 14, 2, 1), (3, 16, 9, 11, 1, 4), (2, 36, 10, 18, 2, 3), (1, 8, 5, 3, 1, 1),
              (2, 20, 40, 24, 2, 2), (40, 32, 28, 28, 1, 1), (2, 64, 30, 32, 1, 2), (2, 24, 6, 20, 2, 1)]


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16])
@pytest.mark.parametrize('case', POOL_CASES, ids=lambda c: 'x'.join(map(str, c)))
def test_spatial_branch_pool(case, dtype):
    """ddf_hip_spatial_branch_pool: the same taps as ddf_hip_spatial_branch, bit for
    bit, and partial sums that add up to the feature planes' sums (the global
    average pool of ddf/ddf.py:184 times H * W)."""
    n, c, h, w_, s, head = case
    torch.manual_seed(7)
    x = torch.randn(n, c, h, w_, device='cuda').to(dtype)
    w = (torch.randn(head * 9, c, device='cuda') * 0.2).to(dtype)
    b = torch.randn(head * 9, device='cuda').to(dtype)
    both = _lib.spatial_branch_pool(x, w, b, head, 3, s, 0.7, None, None)
    assert both is not None
    sf, parts = both
    assert parts.dtype == torch.float32 and parts.shape[0] == n and parts.shape[2] == c
    assert torch.equal(sf, _lib.spatial_branch(x, w, b, head, 3, s, 0.7, None, None))
    sums = x.double().sum((2, 3)).cpu()
    scale = x.double().abs().sum((2, 3)).cpu().max()
    assert ((parts.double().sum(1).cpu() - sums).abs().max() / scale).item() < 1e-6


def test_spatial_branch_pool_turns_down_what_it_cannot_cover():
    x = torch.randn(2, 16, 9, 8, device='cuda')
    w5 = torch.randn(25, 16, device='cuda')
    w3 = torch.randn(9, 16, device='cuda')
    assert _lib.spatial_branch_pool(x, w5, None, 1, 5, 1, 1.0) is None      # 5 x 5 taps
    assert _lib.spatial_branch_pool(x, w3, None, 1, 3, 2, 1.0) is None      # odd height under stride 2
    assert _lib.spatial_branch_pool(x[:, :, :8].contiguous(), w3, None, 1, 3, 2, 1.0) is not None
    assert _lib.spatial_branch_pool(x[:, :15].contiguous(), w3[:, :15].contiguous(), None, 1, 3, 1, 1.0) is None   # odd channel count


@pytest.mark.parametrize('dtype,tol', [(torch.float32, 2e-5), (torch.float16, 6e-3)])
@pytest.mark.parametrize('n,c,k,tiles', [(3, 16, 3, 1), (128, 64, 3, 13), (5, 128, 3, 4), (4, 256, 3, 2),
                                         (3, 512, 3, 7), (2, 70, 5, 3), (19, 160, 3, 1), (128, 512, 3, 4),
                                         (33, 256, 3, 16), (5, 192, 5, 6), (40, 1024, 3, 28)])
def test_channel_branch_parts_matches_fp64(n, c, k, tiles, dtype, tol):
    torch.manual_seed(n + c)
    mid = int(c * 0.2)
    parts = torch.randn(n, tiles, c, device='cuda')
    scale = 1.0 / 37
    w1 = (torch.randn(mid, c, device='cuda') * 0.2).to(dtype)
    b1 = torch.randn(mid, device='cuda').to(dtype)
    w2 = (torch.randn(c * k * k, mid, device='cuda') * 0.3).to(dtype)
    b2 = torch.randn(c * k * k, device='cuda').to(dtype)
    gv = (torch.rand(c * k * k, device='cuda') + 0.5).to(dtype)
    ov = torch.randn(c * k * k, device='cuda').to(dtype)
    out = _lib.channel_branch_parts(parts, scale, w1, b1, w2, b2, k, 1.0, gv, ov)
    assert out.dtype == dtype
    pooled = parts.double().sum(1).cpu() * scale
    ref = channel_reference(pooled, *(t.cpu() for t in (w1, b1, w2, b2)), k, 1.0, gv.cpu(), ov.cpu())
    err = ((out.double().cpu() - ref).abs().max() / ref.abs().max()).item()
    assert err < tol, err
