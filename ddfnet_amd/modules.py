"""Callers of the ``ddf`` operator: filter normalisation, the two filter
branches, ``DDFPack`` and ``DDFUpPack``.

These are ordinary PyTorch modules around the HIP operator.  Constructor
arguments, sub-module names and parameter names follow the reference
(``ddf/ddf.py:125-272``) so that its checkpoints load and its callers
(``ddf_resnet.py:46-47``, ``test_time.py:56``) construct them unchanged.
"""
import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.nn.init import calculate_gain

from . import _lib
from . import functional
from .functional import ddf, ddf_up

__all__ = ['FilterNorm', 'build_spatial_branch', 'build_channel_branch',
           'DDFPack', 'DDFUpPack']


def _standardize(x, dim):
    """(x - mean) / (unbiased std + 1e-10) over ``dim``
    (``ddf/ddf.py:149-150``, ``:162-163``)."""
    var, mean = torch.var_mean(x, dim=dim, keepdim=True)  # unbiased by default
    return (x - mean) / (var.sqrt() + 1e-10)


class _FilterNormFunction(torch.autograd.Function):
    """``gain * standardised(x) + offset`` over the taps of an
    ``(outer, groups, taps, inner)`` tensor, forward and backward one launch each."""

    @staticmethod
    def forward(ctx, x, gain_vec, offset_vec, outer, groups, taps, inner, gain):
        x = x.contiguous()
        ctx.save_for_backward(x, gain_vec)
        ctx.dims = (outer, groups, taps, inner)
        ctx.gain = gain
        return _lib.filter_norm(x, outer, groups, taps, inner, gain, gain_vec, offset_vec)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_y):
        x, gain_vec = ctx.saved_tensors
        outer, groups, taps, inner = ctx.dims
        grad_y = grad_y.to(x.dtype).contiguous()
        want_gain = gain_vec is not None and ctx.needs_input_grad[1]
        grad_x, terms = _lib.filter_norm_backward(grad_y, x, outer, groups, taps, inner, ctx.gain,
                                                  gain_vec, want_gain)
        grad_gain = grad_offset = None
        if want_gain:
            grad_gain = terms.view(outer, groups, taps, inner).sum(dim=(0, 3)).reshape(-1)
        if ctx.needs_input_grad[2]:
            grad_offset = grad_y.view(outer, groups, taps, inner).sum(dim=(0, 3)).reshape(-1)
        if not ctx.needs_input_grad[0]:
            grad_x = None
        return grad_x, grad_gain, grad_offset, None, None, None, None, None


class FilterNorm(nn.Module):
    """Standardise every predicted filter over its ``kernel_size**2`` taps, then
    scale by a gain: the constant ``calculate_gain(nonlinearity) / kernel_size``
    or, with ``running_std``, a learned per-tap vector initialised around it;
    ``running_mean`` adds a learned per-tap offset (``ddf/ddf.py:125-173``).

    ``'spatial'`` input is ``(b, in_channels * k*k, h, w)`` with taps on dim 1;
    ``'channel'`` input is anything reshapeable to ``(b, in_channels, k*k)``
    and comes back as ``(b, in_channels * k*k)``.
    """

    def __init__(self, in_channels, kernel_size, filter_type,
                 nonlinearity='linear', running_std=False, running_mean=False):
        assert filter_type in ('spatial', 'channel')
        assert in_channels >= 1
        super(FilterNorm, self).__init__()
        self.in_channels = in_channels
        self.filter_type = filter_type
        # attribute spellings kept from the reference (ddf/ddf.py:133-134)
        self.runing_std = running_std
        self.runing_mean = running_mean
        taps = in_channels * kernel_size ** 2
        gain = calculate_gain(nonlinearity) / kernel_size
        self.std = nn.Parameter(torch.randn(taps) * gain) if running_std else gain
        if running_mean:
            self.mean = nn.Parameter(torch.randn(taps))

    def _affine(self, x, shape):
        x = x * (self.std.view(shape) if self.runing_std else self.std)
        if self.runing_mean:
            x = x + self.mean.view(shape)
        return x

    def _fused(self, x, outer, inner):
        """One HIP launch instead of the chain of elementwise ops below (and one
        more for its gradient, instead of what autograd derives from the chain)."""
        taps = x.numel() // max(outer * self.in_channels * inner, 1)
        gain_vec = self.std.to(x.dtype) if self.runing_std else None
        offset_vec = self.mean.to(x.dtype) if self.runing_mean else None
        gain = 1.0 if self.runing_std else self.std
        return _FilterNormFunction.apply(x, gain_vec, offset_vec, outer, self.in_channels, taps,
                                         inner, gain)

    def _use_fused(self, x):
        return x.is_cuda and x.dtype in _lib.DTYPE and x.numel() > 0

    def forward(self, x):
        if self._use_fused(x):
            if self.filter_type == 'spatial':
                b, ch, h, w = x.size()
                return self._fused(x, b, h * w).reshape(b, ch, h, w)
            b = x.size(0)
            return self._fused(x.reshape(b, -1), b, 1)
        if self.filter_type == 'spatial':
            b, ch, h, w = x.size()
            x = _standardize(x.reshape(b, self.in_channels, -1, h, w), 2)
            return self._affine(x.reshape(b, ch, h, w), (1, -1, 1, 1))
        if self.filter_type == 'channel':
            b = x.size(0)
            x = _standardize(x.reshape(b, self.in_channels, -1), 2)
            return self._affine(x.reshape(b, -1), (1, -1))
        raise RuntimeError('Unsupported filter type {}'.format(self.filter_type))


def _unhooked(module):
    """No forward / backward hook is registered on the module."""
    return not (module._forward_hooks or module._forward_pre_hooks or module._backward_hooks or
                getattr(module, '_backward_pre_hooks', None))


def _plain_pointwise_conv(module, stride):
    """A 1x1 nn.Conv2d that is a matrix product per (strided) pixel: no groups,
    padding or dilation, nothing hooked."""
    return (type(module) is nn.Conv2d and _unhooked(module) and module.kernel_size == (1, 1) and
            module.stride == (stride, stride) and module.padding == (0, 0) and
            module.dilation == (1, 1) and module.groups == 1 and module.padding_mode == 'zeros')


def build_spatial_branch(in_channels, kernel_size, head=1,
                         nonlinearity='relu', stride=1):
    """1x1 convolution (strided like the operator) to ``head * k*k`` taps per
    pixel, then FilterNorm (``ddf/ddf.py:176-180``)."""
    return nn.Sequential(
        nn.Conv2d(in_channels, head * kernel_size ** 2, 1, stride=stride),
        FilterNorm(head, kernel_size, 'spatial', nonlinearity))


def build_channel_branch(in_channels, kernel_size,
                         nonlinearity='relu', se_ratio=0.2):
    """Squeeze-and-excite style branch: global average pool, bottleneck MLP of
    1x1 convolutions, FilterNorm with a learned gain (``ddf/ddf.py:183-192``)."""
    assert se_ratio > 0
    mid_channels = int(in_channels * se_ratio)
    return nn.Sequential(
        nn.AdaptiveAvgPool2d((1, 1)),
        nn.Conv2d(in_channels, mid_channels, 1),
        nn.ReLU(True),
        nn.Conv2d(mid_channels, in_channels * kernel_size ** 2, 1),
        FilterNorm(in_channels, kernel_size, 'channel', nonlinearity, running_std=True))


class DDFPack(nn.Module):
    """Replacement for a ``k x k`` convolution: predicts both filters from the
    input and applies them with ``ddf`` (``ddf/ddf.py:195-222``).  ``head > 1``
    splits the channels into groups that each get their own spatial filter."""

    def __init__(self, in_channels, kernel_size=3, stride=1, dilation=1, head=1,
                 se_ratio=0.2, nonlinearity='relu', kernel_combine='mul'):
        super(DDFPack, self).__init__()
        assert kernel_size > 1
        self.kernel_size = kernel_size
        self.stride = stride
        self.dilation = dilation
        self.head = head
        self.kernel_combine = kernel_combine
        # (training: normalisation + operator as one autograd node; off = op by op)
        self.fuse_spatial_norm = True
        # inference: the global average pool rides on the spatial branch's launch
        self.fuse_pool = True
        self.spatial_branch = build_spatial_branch(
            in_channels, kernel_size, head, nonlinearity, stride)
        self.channel_branch = build_channel_branch(
            in_channels, kernel_size, nonlinearity, se_ratio)

    def _stock_channel_branch(self):
        """The channel branch is exactly what build_channel_branch makes (global
        average pool, plain 1x1 convolution, ReLU, plain 1x1 convolution,
        FilterNorm) and nothing listens on its modules."""
        branch = self.channel_branch
        return (isinstance(branch, nn.Sequential) and len(branch) == 5 and _unhooked(branch) and
                isinstance(branch[0], nn.AdaptiveAvgPool2d) and _unhooked(branch[0]) and
                branch[0].output_size in (1, (1, 1)) and
                _plain_pointwise_conv(branch[1], 1) and
                type(branch[2]) is nn.ReLU and _unhooked(branch[2]) and
                _plain_pointwise_conv(branch[3], 1) and
                type(branch[4]) is FilterNorm and _unhooked(branch[4]) and
                branch[4].filter_type == 'channel')

    def _stock_spatial_branch(self):
        branch = self.spatial_branch
        return (isinstance(branch, nn.Sequential) and len(branch) == 2 and _unhooked(branch) and
                _plain_pointwise_conv(branch[0], self.stride) and
                type(branch[1]) is FilterNorm and _unhooked(branch[1]) and
                branch[1].filter_type == 'spatial' and branch[1].in_channels == self.head)

    def _channel_filter(self, x):
        """The channel branch.  Its two 1x1 convolutions act on a pooled
        (b, c, 1, 1) tensor, i.e. they are matrix products: evaluating them as
        such (same parameters, same arithmetic) avoids the convolution
        library's launch path, which costs more host time than the whole layer
        has GPU work at small feature maps."""
        branch = self.channel_branch
        if not (x.is_cuda and self._stock_channel_branch()):
            return branch(x)   # not the stock branch: run it as it is
        fc1, fc2, norm = branch[1], branch[3], branch[4]
        v = x.mean((2, 3))
        v = F.relu(F.linear(v, fc1.weight.flatten(1), fc1.bias))
        return norm(F.linear(v, fc2.weight.flatten(1), fc2.bias))

    def _inference_filters(self, x):
        """Both filters with one launch per branch (plus the pooling) - or, with
        the torch extension, the layer's result itself - or None where that
        path does not apply: gradients wanted, branches that are not
        the stock ones, a dtype or kernel size the branch kernels lack, or
        parameters in another dtype than the features (autocast)."""
        if torch.is_grad_enabled() and (x.requires_grad or
                                        any(p.requires_grad for p in self.parameters())):
            return None
        k = self.kernel_size
        # (a size the stride does not divide: the op-by-op path fails at its reshape, as the
        # reference does at ddf/ddf.py:215-218, and so must this one)
        if x.dim() == 4 and (x.size(2) % self.stride or x.size(3) % self.stride):
            return None
        if not (x.is_cuda and x.dim() == 4 and _lib.branches_cover(k, x.dtype) and
                self._stock_channel_branch() and self._stock_spatial_branch()):
            return None
        conv, sp_norm = self.spatial_branch
        fc1, fc2, ch_norm = self.channel_branch[1], self.channel_branch[3], self.channel_branch[4]
        tensors = [conv.weight, conv.bias, fc1.weight, fc1.bias, fc2.weight, fc2.bias]
        for norm in (sp_norm, ch_norm):
            tensors += [norm.std if norm.runing_std else None,
                        norm.mean if norm.runing_mean else None]
        if any(t is not None and (t.dtype != x.dtype or t.device != x.device) for t in tensors):
            return None
        if ch_norm.in_channels != x.size(1) or fc1.in_channels != x.size(1):
            return None
        ext = functional.extension()
        if ext is not None:
            # the same launches without the interpreter in between
            return ext.ddf_pack_forward(
                x, conv.weight, conv.bias,
                1.0 if sp_norm.runing_std else sp_norm.std, tensors[6], tensors[7],
                fc1.weight, fc1.bias, fc2.weight, fc2.bias,
                1.0 if ch_norm.runing_std else ch_norm.std, tensors[8], tensors[9],
                k, self.dilation, self.stride, self.head, self.kernel_combine, self.fuse_pool)
        x = x.contiguous()
        ch_args = (fc1.weight, fc1.bias, fc2.weight, fc2.bias, k,
                   1.0 if ch_norm.runing_std else ch_norm.std,
                   ch_norm.std if ch_norm.runing_std else None,
                   ch_norm.mean if ch_norm.runing_mean else None)
        sp_args = (conv.weight, conv.bias, self.head, k, self.stride,
                   1.0 if sp_norm.runing_std else sp_norm.std,
                   sp_norm.std if sp_norm.runing_std else None,
                   sp_norm.mean if sp_norm.runing_mean else None)
        # the spatial branch reads every feature plane anyway: where its kernel can, it
        # leaves the planes' partial sums and the channel branch pools from those
        pooled = _lib.spatial_branch_pool(x, *sp_args) if self.fuse_pool else None
        if pooled is not None:
            sf, parts = pooled
            return _lib.channel_branch_parts(parts, 1.0 / (x.size(2) * x.size(3)), *ch_args), sf
        cf = _lib.channel_branch(x.mean((2, 3)), *ch_args)
        sf = _lib.spatial_branch(x, *sp_args)
        return cf, sf

    def forward(self, x):
        b, c, h, w = x.shape
        g, k, s = self.head, self.kernel_size, self.stride
        ho, wo = h // s, w // s
        filters = self._inference_filters(x)
        if torch.is_tensor(filters):      # the whole layer was run
            return filters
        if filters is not None:
            cf, sf = filters
            out = ddf(x.reshape(b * g, c // g, h, w), cf.reshape(b * g, c // g, k, k),
                      sf.reshape(b * g, k * k, ho, wo), k, self.dilation, s, self.kernel_combine)
            return out.reshape(b, c, ho, wo)
        cf = self._channel_filter(x).reshape(b * g, c // g, k, k)
        if self.fuse_spatial_norm and x.is_cuda and self._stock_spatial_branch() and \
                not self.spatial_branch[1].runing_mean and h % s == 0 and w % s == 0:
            # Training: the spatial filter normalisation and the operator as one autograd
            # node, whose backward pushes dSF through the normalisation in the launch that
            # adds up the filter gradients' partial sums (no launch of its own for the
            # normalisation's gradient, no round trip of dSF through memory).
            conv, norm = self.spatial_branch
            raw = conv(x).reshape(b * g, k * k, ho, wo)
            out = functional.ddf_spatial_norm(
                x.reshape(b * g, c // g, h, w), cf, raw, k, self.dilation, s, self.kernel_combine,
                g, 1.0 if norm.runing_std else norm.std, norm.std if norm.runing_std else None)
            return out.reshape(b, c, ho, wo)
        sf = self.spatial_branch(x).reshape(b * g, k * k, ho, wo)
        out = ddf(x.reshape(b * g, c // g, h, w), cf, sf,
                  k, self.dilation, s, self.kernel_combine)
        return out.reshape(b, c, ho, wo)


class DDFUpPack(nn.Module):
    """Upsampling pack: ``scale_factor**2`` (spatial, channel) branch pairs, one
    ``ddf`` call per pair, outputs interleaved by pixel shuffle
    (``ddf/ddf.py:225-272``).  The spatial filters may be predicted from a
    separate guidance tensor ``joint_x``.

    The reference's ``forward`` passes ``self.head`` in the ``kernel_combine``
    position (``ddf/ddf.py:267-268``) and so trips the operator's own
    assertion; here the arguments are in the operator's order.
    """

    def __init__(self, in_channels, kernel_size=3, scale_factor=2, dilation=1, head=1, se_ratio=0.2,
                 nonlinearity='linear', dw_kernel_size=3, joint_channels=-1, kernel_combine='mul'):
        super(DDFUpPack, self).__init__()
        self.kernel_size = kernel_size
        self.dilation = dilation
        self.head = head
        self.scale_factor = scale_factor
        self.kernel_combine = kernel_combine

        self.spatial_branch = nn.ModuleList()
        self.channel_branch = nn.ModuleList()
        own_guidance = joint_channels < 1
        if own_guidance:
            dw_kernel_size = max(dw_kernel_size, 3)
        for _ in range(scale_factor ** 2):
            spatial = build_spatial_branch(in_channels, kernel_size, head, nonlinearity, 1)
            if own_guidance:
                # a depthwise convolution first gives each sub-pixel branch its
                # own view of the neighbourhood
                spatial = nn.Sequential(
                    nn.Conv2d(in_channels, in_channels, dw_kernel_size,
                              padding=kernel_size // 2, groups=in_channels),
                    spatial)
            self.spatial_branch.append(spatial)
            self.channel_branch.append(
                build_channel_branch(in_channels, kernel_size, nonlinearity, se_ratio))

    def forward(self, x, joint_x=None):
        if joint_x is None:
            joint_x = x
        b, c, h, w = x.shape
        g, k = self.head, self.kernel_size
        r = self.scale_factor
        grouped = x.reshape(b * g, c // g, h, w)
        cfs = [channel(x).reshape(b * g, c // g, k, k) for channel in self.channel_branch]
        sfs = [spatial(joint_x).reshape(b * g, k * k, h, w) for spatial in self.spatial_branch]
        # all r*r branches, the stack and the pixel shuffle as one operator
        out = ddf_up(grouped, cfs, sfs, k, self.dilation, r, self.kernel_combine)
        return out.type_as(x).reshape(b, c, h * r, w * r)
