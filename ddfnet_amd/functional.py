"""The ``ddf`` autograd operator on the gfx950 HIP kernels.

Host-side mirror of ``DDFFunction`` / ``ddf`` / ``OP_DICT`` of the reference
(``ddf/ddf.py:19-122``): same positional signature, same assertion messages,
same 8-tuple from ``backward``.  All arithmetic of the operator happens in
``libddf_hip.so``; nothing here computes it in PyTorch and there is no
fallback when the library is missing.

Deliberate differences from the reference, each a superset of its behaviour:

* fp16 runs natively (fp16 in and out, fp32 accumulation) rather than being
  widened to fp32 first (``ddf/ddf.py:36-42``, ``:74``).  Operands of different
  dtypes are promoted to the widest one, which is what the reference's
  per-tensor widening amounts to.
* Non-contiguous operands are made contiguous instead of raising
  (``ddf/src/cuda/ddf_mul_cuda.cpp:27-32``).
* Only the gradients autograd asks for are computed, and none of the six
  zero-filled tensors of ``ddf/ddf.py:106-111`` is allocated.
"""
import torch
from torch.autograd import Function

from . import _lib

__all__ = ['DDFFunction', 'ddf', 'OP_DICT', 'DDFUpFunction', 'ddf_up', 'DDFSpatialNormFunction',
           'ddf_spatial_norm']


def _require_device_contiguous(named_tensors):
    """What CHECK_INPUT enforces in ddf/src/cuda/ddf_mul_cuda.cpp:25-32, and the
    CPU rejection of ddf/src/ddf_mul_ext.cpp:33."""
    for name, t in named_tensors:
        if t is None:
            continue
        if not t.is_cuda:
            if name in ('features', 'top_grad'):
                raise RuntimeError('ddf operation is not implemented on CPU')
            raise RuntimeError(name + ' must be a CUDA tensor ')
        if not t.is_contiguous():
            raise RuntimeError(name + ' must be contiguous ')


class _NativeOp(object):
    """Stand-in for one of the reference's four extension modules
    (``ddf/src/ddf_mul_ext.cpp:57-60``, ``ddf_mul_faster_ext.cpp:28-30``):
    caller-allocated outputs, positional arguments in the reference's order,
    return value 1."""

    def __init__(self, combine, variant, with_backward=True):
        self.combine, self.variant = combine, variant
        if not with_backward:  # the faster modules export forward only
            self.backward = None

    def forward(self, features, channel_filter, spatial_filter,
                kernel_size, dilation, stride, output):
        _require_device_contiguous((('features', features),
                                    ('channel_filter', channel_filter),
                                    ('spatial_filter', spatial_filter),
                                    ('output', output)))
        with _lib.on_device_of(features):
            _lib.forward(features, channel_filter, spatial_filter, output,
                         kernel_size, dilation, stride, self.combine, self.variant)
        return 1

    def backward(self, top_grad, features, channel_filter, spatial_filter,
                 kernel_size, dilation, stride,
                 rtop_grad, rbottom_grad, rspatial_filter_grad,
                 bottom_grad, channel_filter_grad, spatial_filter_grad):
        """``rtop_grad``, ``rbottom_grad`` and ``rspatial_filter_grad`` were
        NHWC scratch in the reference (``ddf/src/cuda/ddf_mul_cuda.cpp:82-87``);
        they are accepted and never touched.  A gradient passed as ``None`` is
        not computed."""
        grads = (('bottom_grad', bottom_grad, _lib.NEED_DX),
                 ('channel_filter_grad', channel_filter_grad, _lib.NEED_DCF),
                 ('spatial_filter_grad', spatial_filter_grad, _lib.NEED_DSF))
        _require_device_contiguous((('top_grad', top_grad), ('features', features),
                                    ('channel_filter', channel_filter),
                                    ('spatial_filter', spatial_filter)) +
                                   tuple((n, t) for n, t, _ in grads))
        need = sum(bit for _, t, bit in grads if t is not None)
        with _lib.on_device_of(features):
            nbytes = _lib.backward_workspace_bytes(
                features.shape, kernel_size, dilation, stride, self.combine,
                features.dtype, need, self.variant)
            workspace = (torch.empty(nbytes, dtype=torch.uint8, device=features.device)
                         if nbytes else None)
            _lib.backward(top_grad, features, channel_filter, spatial_filter,
                          bottom_grad, channel_filter_grad, spatial_filter_grad,
                          kernel_size, dilation, stride, self.combine, need,
                          workspace, self.variant)
        return 1


# Keys as in ddf/ddf.py:19-24.  The '*_faster' entries force the tiled kernels.
OP_DICT = {
    'mul': _NativeOp('mul', ''),
    'mul_faster': _NativeOp('mul', 'f', with_backward=False),
    'add': _NativeOp('add', ''),
    'add_faster': _NativeOp('add', 'f', with_backward=False),
}
# version='o': the generic kernels, forward and backward.
_ORIGINAL = {'mul': _NativeOp('mul', 'o'), 'add': _NativeOp('add', 'o')}


class DDFFunction(Function):
    @staticmethod
    def forward(ctx, features, channel_filter, spatial_filter,
                kernel_size=3, dilation=1, stride=1, kernel_combine='mul', version=''):
        assert features.is_cuda, 'input feature must be a CUDA tensor.'
        assert channel_filter.is_cuda, 'channel_filter must be a CUDA tensor.'
        assert spatial_filter.is_cuda, 'spatial_filter must be a CUDA tensor.'

        # one working dtype for the three operands
        dtype = features.dtype
        for other in (channel_filter, spatial_filter):
            dtype = torch.promote_types(dtype, other.dtype)
        assert dtype in _lib.DTYPE, 'unsupported dtype {}'.format(dtype)
        features, channel_filter, spatial_filter = (
            t.to(dtype).contiguous() for t in (features, channel_filter, spatial_filter))

        b, c, h, w = features.size()
        out_h, out_w = h // stride, w // stride
        bc, cc, hc, wc = channel_filter.size()
        assert bc == b and cc == c,\
            "channel_filter size {} does not match feature size {}".format(
                channel_filter.size(), features.size())
        assert hc == kernel_size and wc == kernel_size,\
            "channel_filter size {} does not match kernel size {}".format(
                channel_filter.size(), kernel_size)
        bs, cs, hs, ws = spatial_filter.size()
        assert bs == b and hs == out_h and ws == out_w,\
            "spatial_filter size {} does not match feature size {} with stride {}".format(
                spatial_filter.size(), features.size(), stride)
        assert cs == kernel_size ** 2,\
            "spatial_filter size {} does not match kernel size {}".format(
                spatial_filter.size(), kernel_size)
        assert (kernel_size - 1) % 2 == 0 and kernel_size >= 1 and dilation >= 1 and stride >= 1
        assert kernel_combine in {'mul', 'add'}, \
            'only support mul or add combination, instead of {}'.format(kernel_combine)
        assert version in {'', 'o', 'f'}, \
            "version must be '', 'o' or 'f', instead of {}".format(version)

        ctx.kernel_size, ctx.dilation, ctx.stride = kernel_size, dilation, stride
        ctx.op_type = kernel_combine
        ctx.version = version

        # 'f' forces the tiled kernels, 'o' the generic ones, '' lets the
        # library choose (the reference's own rule is at ddf/ddf.py:77-84).
        if version == 'f':
            op = OP_DICT[kernel_combine + '_faster']
        elif version == 'o':
            op = _ORIGINAL[kernel_combine]
        else:
            op = OP_DICT[kernel_combine]

        # the kernels write every element, so no zero fill
        output = features.new_empty((b, c, out_h, out_w))
        op.forward(features, channel_filter, spatial_filter,
                   kernel_size, dilation, stride, output)
        # (asked of ctx, not of the tensors: a dtype or layout conversion above
        # yields new tensors that no longer carry the inputs' requires_grad)
        if any(ctx.needs_input_grad[:3]):
            ctx.save_for_backward(features, channel_filter, spatial_filter)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        assert grad_output.is_cuda
        features, channel_filter, spatial_filter = ctx.saved_tensors
        grad_output = grad_output.to(features.dtype).contiguous()

        wanted = ctx.needs_input_grad[:3]
        grad_input, grad_channel_filter, grad_spatial_filter = (
            torch.empty_like(t) if w else None
            for t, w in zip((features, channel_filter, spatial_filter), wanted))

        op = _ORIGINAL[ctx.op_type] if ctx.version == 'o' else OP_DICT[ctx.op_type]
        op.backward(grad_output, features, channel_filter, spatial_filter,
                    ctx.kernel_size, ctx.dilation, ctx.stride, None, None, None,
                    grad_input, grad_channel_filter, grad_spatial_filter)
        return grad_input, grad_channel_filter, grad_spatial_filter, None, None, None, None, None


# The operator callers use: the C++ autograd function of the torch extension
# (csrc/torch/ddf_torch.cpp: same checks, same messages, same library calls,
# without the interpreter in between) where it has been built, else the Python
# Function above.  Both enqueue the same kernels.  The extension is looked up at
# the first call rather than at import, so a process that imports the package
# and builds the extension afterwards still picks it up.
_C = None
_C_missing = False


def extension(retry=False):
    """The torch extension module ``ddfnet_amd._C``, or None where it (or the
    library it links) has not been built.  ``retry`` looks again after a miss."""
    global _C, _C_missing
    if _C is None and (retry or not _C_missing):
        try:
            import importlib
            importlib.invalidate_caches()
            _C = importlib.import_module(__package__ + '._C')
        except ImportError:      # extension (or the library it links) not built
            _C_missing = True
    return _C


_DDF_ARGS = ('features', 'channel_filter', 'spatial_filter', 'kernel_size', 'dilation', 'stride',
             'kernel_combine', 'version')
_DDF_DEFAULTS = {'kernel_size': 3, 'dilation': 1, 'stride': 1, 'kernel_combine': 'mul', 'version': ''}


def ddf(*args, **kwargs):
    """The operator, ``DDFFunction.apply`` of ``ddf/ddf.py:122``; arguments may
    also be given by the names of ``DDFFunction.forward``."""
    ext = extension()
    if ext is not None:
        return ext.ddf(*args, **kwargs)
    if kwargs:
        named = dict(_DDF_DEFAULTS)
        named.update(zip(_DDF_ARGS, args))
        for name in kwargs:
            if name not in _DDF_ARGS or name in _DDF_ARGS[:len(args)]:
                raise TypeError("ddf() got an unexpected or repeated argument '%s'" % name)
        named.update(kwargs)
        args = tuple(named[name] for name in _DDF_ARGS)
    return DDFFunction.apply(*args)


class DDFSpatialNormFunction(Function):
    """``ddf(features, channel_filter, FilterNorm(raw_spatial_filter), ...)`` as
    one autograd node: the spatial filter normalisation of ``DDFPack``
    (``ddf/ddf.py:146-157``, constant or learned per-tap gain, no offset) in
    front of the operator (``ddf/ddf.py:217-221``).

    Forward: the normalisation launch, then the operator's.  Backward: one
    library call in which the launch that adds up the filter gradients' partial
    sums also applies the normalisation's Jacobian, so the gradient of the
    normalised filter is never written to memory and the normalisation's
    gradient costs no launch of its own.

    ``raw_spatial_filter`` is ``(b * groups, k*k, h // s, w // s)`` as the
    operator takes it (``groups`` = the layer's ``head``: sample ``n`` uses row
    ``n % groups`` of ``gain_vec``)."""

    @staticmethod
    def forward(ctx, features, channel_filter, raw_spatial_filter, gain_vec, kernel_size, dilation,
                stride, kernel_combine, groups, gain):
        assert features.is_cuda and channel_filter.is_cuda and raw_spatial_filter.is_cuda
        assert kernel_combine in {'mul', 'add'}, \
            'only support mul or add combination, instead of {}'.format(kernel_combine)
        dtype = torch.promote_types(torch.promote_types(features.dtype, channel_filter.dtype),
                                    raw_spatial_filter.dtype)
        assert dtype in _lib.DTYPE, 'unsupported dtype {}'.format(dtype)
        features = features.to(dtype).contiguous()
        channel_filter = channel_filter.to(dtype).contiguous()
        raw = raw_spatial_filter.to(dtype).contiguous()
        gain_vec = None if gain_vec is None else gain_vec.to(dtype).contiguous()
        b, c, h, w = features.size()
        k = kernel_size
        assert tuple(channel_filter.size()) == (b, c, k, k), \
            "channel_filter size {} does not match feature size {}".format(
                channel_filter.size(), features.size())
        assert tuple(raw.size()) == (b, k * k, h // stride, w // stride), \
            "spatial_filter size {} does not match feature size {}".format(
                raw.size(), features.size())
        assert groups >= 1 and b % groups == 0
        ho, wo = h // stride, w // stride
        with _lib.on_device_of(features):
            spatial_filter = _lib.filter_norm(raw, b // groups, groups, k * k, ho * wo, gain, gain_vec)
            output = features.new_empty((b, c, ho, wo))
            _lib.forward(features, channel_filter, spatial_filter, output, k, dilation, stride,
                         kernel_combine, '')
        ctx.conf = (k, dilation, stride, kernel_combine, groups, gain)
        if any(ctx.needs_input_grad):
            ctx.save_for_backward(features, channel_filter, spatial_filter, raw, gain_vec)
        return output

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_output):
        features, channel_filter, spatial_filter, raw, gain_vec = ctx.saved_tensors
        k, d, s, combine, groups, gain = ctx.conf
        grad_output = grad_output.to(features.dtype).contiguous()
        want = ctx.needs_input_grad
        want_gain = gain_vec is not None and want[3]
        need = ((_lib.NEED_DX if want[0] else 0) | (_lib.NEED_DCF if want[1] else 0) |
                (_lib.NEED_DSF if (want[2] or want_gain) else 0))
        gx = torch.empty_like(features) if want[0] else None
        gcf = torch.empty_like(channel_filter) if want[1] else None
        graw = torch.empty_like(raw) if need & _lib.NEED_DSF else None
        terms = torch.empty_like(raw) if want_gain else None
        if need:
            with _lib.on_device_of(features):
                _lib.backward_spatial_norm(grad_output, features, channel_filter, spatial_filter,
                                           raw, gx, gcf, graw, terms, k, d, s, combine, need,
                                           groups, gain, gain_vec)
        ggain = None
        if want_gain:
            b, kk, ho, wo = raw.shape
            ggain = terms.view(b // groups, groups, kk, ho * wo).sum(dim=(0, 3)).reshape(-1)
        return gx, gcf, (graw if want[2] else None), ggain, None, None, None, None, None, None


def ddf_spatial_norm(features, channel_filter, raw_spatial_filter, kernel_size=3, dilation=1,
                     stride=1, kernel_combine='mul', groups=1, gain=1.0, gain_vec=None):
    """``ddf`` on the spatial filter ``gain * standardised(raw_spatial_filter)``
    (standardised over the ``kernel_size**2`` taps of every pixel; ``gain_vec``,
    ``(groups * kernel_size**2,)``, replaces the scalar gain)."""
    return DDFSpatialNormFunction.apply(features, channel_filter, raw_spatial_filter, gain_vec,
                                        kernel_size, dilation, stride, kernel_combine, groups, gain)


class DDFUpFunction(Function):
    """Up-sampling DDF: ``scale*scale`` filter branches on the same features,
    result pixel-shuffled -- the loop, ``torch.stack`` and ``F.pixel_shuffle``
    of ``DDFUpPack.forward`` (``ddf/ddf.py:264-272``) as one operator.

    The forward is one launch that reads the features once and writes the
    (N, C, H*scale, W*scale) result in place.  The backward is one library call
    that splits the incoming gradient into its ``scale*scale`` sub-pixel
    lattices, runs the ``ddf`` backward kernels per branch and sums their dX.
    """

    @staticmethod
    def forward(ctx, features, kernel_size, dilation, scale, kernel_combine, *filters):
        branches = scale * scale
        assert len(filters) == 2 * branches, \
            'expected {0} channel filters followed by {0} spatial filters'.format(branches)
        assert features.is_cuda, 'input feature must be a CUDA tensor.'
        assert kernel_combine in {'mul', 'add'}, \
            'only support mul or add combination, instead of {}'.format(kernel_combine)
        assert (kernel_size - 1) % 2 == 0 and kernel_size >= 1 and dilation >= 1
        dtype = features.dtype
        for other in filters:
            assert other.is_cuda, 'filters must be CUDA tensors.'
            dtype = torch.promote_types(dtype, other.dtype)
        assert dtype in _lib.DTYPE, 'unsupported dtype {}'.format(dtype)
        features = features.to(dtype).contiguous()
        filters = [t.to(dtype).contiguous() for t in filters]
        cfs, sfs = filters[:branches], filters[branches:]
        b, c, h, w = features.size()
        for cf in cfs:
            assert tuple(cf.size()) == (b, c, kernel_size, kernel_size), \
                "channel_filter size {} does not match feature size {}".format(
                    cf.size(), features.size())
        for sf in sfs:
            assert tuple(sf.size()) == (b, kernel_size ** 2, h, w), \
                "spatial_filter size {} does not match feature size {}".format(
                    sf.size(), features.size())
        ctx.kernel_size, ctx.dilation, ctx.scale = kernel_size, dilation, scale
        ctx.op_type = kernel_combine

        output = features.new_empty((b, c, h * scale, w * scale))
        with _lib.on_device_of(features):
            _lib.up_forward(features, cfs, sfs, output, kernel_size, dilation, scale,
                            kernel_combine)
        if any(ctx.needs_input_grad):
            ctx.save_for_backward(features, *filters)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        saved = ctx.saved_tensors
        features, filters = saved[0], saved[1:]
        r = ctx.scale
        branches = r * r
        cfs, sfs = filters[:branches], filters[branches:]
        grad_output = grad_output.to(features.dtype).contiguous()
        want_f = ctx.needs_input_grad[5:]
        grad_x = torch.empty_like(features) if ctx.needs_input_grad[0] else None
        grad_cfs = [torch.empty_like(t) if w else None for t, w in zip(cfs, want_f[:branches])]
        grad_sfs = [torch.empty_like(t) if w else None for t, w in zip(sfs, want_f[branches:])]
        with _lib.on_device_of(features):
            _lib.up_backward(grad_output, features, cfs, sfs, grad_x, grad_cfs, grad_sfs,
                             ctx.kernel_size, ctx.dilation, r, ctx.op_type)
        return (grad_x, None, None, None, None) + tuple(grad_cfs) + tuple(grad_sfs)


def ddf_up(features, channel_filters, spatial_filters, kernel_size=3, dilation=1,
           scale_factor=2, kernel_combine='mul'):
    """``pixel_shuffle`` of the ``scale_factor**2`` results ``ddf(features,
    channel_filters[b], spatial_filters[b], kernel_size, dilation, 1,
    kernel_combine)``, branch ``b`` going to sub-pixel ``divmod(b, scale_factor)``.

    One fused launch where the library has a kernel for (kernel_size,
    scale_factor); otherwise the reference's composition (``ddf/ddf.py:264-272``)
    on the ``ddf`` kernels."""
    channel_filters, spatial_filters = tuple(channel_filters), tuple(spatial_filters)
    assert len(channel_filters) == len(spatial_filters) == scale_factor ** 2
    if _lib.up_forward_covers(kernel_size, scale_factor):
        ext = extension()
        if ext is not None:   # the same operator as a C++ autograd function
            return ext.ddf_up(features, list(channel_filters), list(spatial_filters), kernel_size,
                             dilation, scale_factor, kernel_combine)
        return DDFUpFunction.apply(features, kernel_size, dilation, scale_factor, kernel_combine,
                                   *(channel_filters + spatial_filters))
    outs = [ddf(features, cf, sf, kernel_size, dilation, 1, kernel_combine)
            for cf, sf in zip(channel_filters, spatial_filters)]
    b, c, h, w = outs[0].shape
    return torch.nn.functional.pixel_shuffle(torch.stack(outs, dim=2).reshape(b, -1, h, w),
                                             scale_factor)
