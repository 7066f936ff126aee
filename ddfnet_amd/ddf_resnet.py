"""DDF-ResNets: ResNet bottleneck networks whose 3x3 convolutions are DDFPacks.

The reference builds these on timm's ``ResNet`` / ``Bottleneck``
(``ddf_resnet.py:34-111``: ``conv2`` of every bottleneck is replaced by
``DDFPack(width, kernel_size=3, stride, dilation, se_ratio=0.2)``).  timm is not
a dependency here, so the skeleton is spelled out: 7x7/2 stem + BN + ReLU +
3x3/2 max-pool, four stages of bottlenecks (expansion 4, stride on the middle
operator, 1x1/stride + BN projection shortcut), global average pool, linear
classifier.  Parameter counts match the reference's model table
(``README.md:20-23``): 16 843 748 for ddf_mul_resnet50, 28 146 912 for
ddf_mul_resnet101.

Initialisation follows timm 0.4.5's ResNet as recalled: Kaiming-normal (fan-out,
ReLU) for convolutions, BatchNorm weight 1 and bias 0, and - with
``zero_init_last_bn`` (default on, as there) - weight 0 for the last BatchNorm
of every bottleneck.  There is no way to check against timm here; only the
structure is pinned.
"""
import ctypes

import torch
import torch.nn as nn

from .functional import ddf  # noqa: F401  (re-exported: callers time the operator through this module)
from .modules import DDFPack

__all__ = ['DDFBottleneck', 'DDFResNet', 'ddf_mul_resnet50', 'ddf_mul_resnet101',
           'ddf_mul_resnet152', 'ddf_add_resnet50', 'ddf_add_resnet101', 'ddf_add_resnet152',
           'time_ddf_layers']


class DDFBottleneck(nn.Module):
    expansion = 4

    def __init__(self, inplanes, planes, stride=1, downsample=None, dilation=1,
                 se_ratio=0.2, kernel_combine='mul'):
        super(DDFBottleneck, self).__init__()
        width = planes
        outplanes = planes * self.expansion
        self.conv1 = nn.Conv2d(inplanes, width, kernel_size=1, bias=False)
        self.bn1 = nn.BatchNorm2d(width)
        self.act1 = nn.ReLU(inplace=True)
        self.conv2 = DDFPack(width, kernel_size=3, stride=stride, dilation=dilation,
                             se_ratio=se_ratio, kernel_combine=kernel_combine)
        self.bn2 = nn.BatchNorm2d(width)
        self.act2 = nn.ReLU(inplace=True)
        self.conv3 = nn.Conv2d(width, outplanes, kernel_size=1, bias=False)
        self.bn3 = nn.BatchNorm2d(outplanes)
        self.act3 = nn.ReLU(inplace=True)
        self.downsample = downsample

    def forward(self, x):
        shortcut = x if self.downsample is None else self.downsample(x)
        x = self.act1(self.bn1(self.conv1(x)))
        x = self.act2(self.bn2(self.conv2(x)))
        x = self.bn3(self.conv3(x))
        return self.act3(x + shortcut)


class DDFResNet(nn.Module):
    def __init__(self, layers, kernel_combine='mul', num_classes=1000, in_chans=3, se_ratio=0.2,
                 zero_init_last_bn=True):
        """``zero_init_last_bn``: start every residual branch at zero by zeroing the
        weight of each block's last BatchNorm (the default of the ResNet the
        reference derives its models from), so a freshly built network is the
        identity on its shortcuts."""
        super(DDFResNet, self).__init__()
        self.num_classes = num_classes
        self.conv1 = nn.Conv2d(in_chans, 64, kernel_size=7, stride=2, padding=3, bias=False)
        self.bn1 = nn.BatchNorm2d(64)
        self.act1 = nn.ReLU(inplace=True)
        self.maxpool = nn.MaxPool2d(kernel_size=3, stride=2, padding=1)
        inplanes = 64
        stages = []
        for i, (planes, blocks) in enumerate(zip((64, 128, 256, 512), layers)):
            stride = 1 if i == 0 else 2
            downsample = None
            if stride != 1 or inplanes != planes * DDFBottleneck.expansion:
                downsample = nn.Sequential(
                    nn.Conv2d(inplanes, planes * DDFBottleneck.expansion, 1, stride=stride,
                              bias=False),
                    nn.BatchNorm2d(planes * DDFBottleneck.expansion))
            blocks_ = [DDFBottleneck(inplanes, planes, stride, downsample, se_ratio=se_ratio,
                                     kernel_combine=kernel_combine)]
            inplanes = planes * DDFBottleneck.expansion
            blocks_ += [DDFBottleneck(inplanes, planes, se_ratio=se_ratio,
                                      kernel_combine=kernel_combine) for _ in range(1, blocks)]
            stages.append(nn.Sequential(*blocks_))
        self.layer1, self.layer2, self.layer3, self.layer4 = stages
        self.global_pool = nn.AdaptiveAvgPool2d(1)
        self.fc = nn.Linear(512 * DDFBottleneck.expansion, num_classes)
        for m in self.modules():
            if isinstance(m, nn.Conv2d):
                nn.init.kaiming_normal_(m.weight, mode='fan_out', nonlinearity='relu')
            elif isinstance(m, nn.BatchNorm2d):
                nn.init.ones_(m.weight)
                nn.init.zeros_(m.bias)
        if zero_init_last_bn:
            for m in self.modules():
                if isinstance(m, DDFBottleneck):
                    nn.init.zeros_(m.bn3.weight)

    def forward_features(self, x):
        x = self.maxpool(self.act1(self.bn1(self.conv1(x))))
        return self.layer4(self.layer3(self.layer2(self.layer1(x))))

    def forward(self, x):
        x = self.global_pool(self.forward_features(x)).flatten(1)
        return self.fc(x)


def _make(layers, combine):
    def build(pretrained=False, **kwargs):
        assert not pretrained, 'no pretrained weights ship with this package'
        return DDFResNet(layers, kernel_combine=combine, **kwargs)
    return build


ddf_mul_resnet50 = _make([3, 4, 6, 3], 'mul')
ddf_mul_resnet101 = _make([3, 4, 23, 3], 'mul')
ddf_mul_resnet152 = _make([3, 8, 36, 3], 'mul')
ddf_add_resnet50 = _make([3, 4, 6, 3], 'add')
ddf_add_resnet101 = _make([3, 4, 23, 3], 'add')
ddf_add_resnet152 = _make([3, 8, 36, 3], 'add')


def fold_batchnorm(model):
    """A copy of an eval-mode ``DDFResNet`` for inference with every BatchNorm
    that directly follows a convolution folded into that convolution's weights and
    bias (the stem's, ``bn1`` and ``bn3`` of each block, the shortcut's).  In eval
    mode BatchNorm is a per-channel affine map, so the network computes the same
    function; ``bn2`` follows the dynamic filter and stays."""
    import copy
    from torch.nn.utils.fusion import fuse_conv_bn_eval
    assert not model.training, 'fold_batchnorm is for eval-mode models'
    model = copy.deepcopy(model)
    model.conv1, model.bn1 = fuse_conv_bn_eval(model.conv1, model.bn1), nn.Identity()
    for block in model.modules():
        if isinstance(block, DDFBottleneck):
            block.conv1, block.bn1 = fuse_conv_bn_eval(block.conv1, block.bn1), nn.Identity()
            block.conv3, block.bn3 = fuse_conv_bn_eval(block.conv3, block.bn3), nn.Identity()
            if block.downsample is not None:
                block.downsample = nn.Sequential(
                    fuse_conv_bn_eval(block.downsample[0], block.downsample[1]))
    return model


def time_ddf_layers(model, x, iters=100, cache_bytes=256 * 1024 * 1024):
    """Run ``model(x)`` once, record the operands of every ``ddf`` call made by
    its DDFPacks, then time each call on its own: the library's forward entry
    point on preallocated results, rotating over enough copies of the operands
    to exceed twice ``cache_bytes`` (the last-level cache), so that the figure is
    a memory figure and not a cache one.  Returns one dict per layer with shape,
    milliseconds and achieved GB/s (algorithmic forward bytes)."""
    from . import _lib
    records = []

    def hook(mod, inputs):
        inp = inputs[0]
        b, c, h, w = inp.shape
        g, k, s = mod.head, mod.kernel_size, mod.stride
        cf = mod.channel_branch(inp).reshape(b * g, c // g, k, k)
        sf = mod.spatial_branch(inp).reshape(b * g, k * k, h // s, w // s)
        records.append((inp.reshape(b * g, c // g, h, w), cf, sf, k, mod.dilation, s,
                        mod.kernel_combine))

    handles = [m.register_forward_pre_hook(hook) for m in model.modules()
               if isinstance(m, DDFPack)]
    with torch.no_grad():
        model(x)
    for h in handles:
        h.remove()
    out = []
    with torch.no_grad():
        for feat, cf, sf, k, d, s, combine in records:
            n, c, h, w = feat.shape
            esz = feat.element_size()
            nbytes = esz * (feat.numel() + n * c * (h // s) * (w // s) + cf.numel() + sf.numel())
            free = torch.cuda.mem_get_info()[0]
            copies = int(max(2, min(2 * cache_bytes // nbytes + 1, (free // 2) // nbytes)))
            sets = [(feat.clone(), cf.clone(), sf.clone(), feat.new_empty((n, c, h // s, w // s)))
                    for _ in range(copies)]
            with _lib.on_device_of(feat):
                # (argument lists built once: the timed loop is the library's entry point
                # and nothing else, or the 10 us kernels of the late stages would be timed
                # at the pace of the Python around them)
                launch = _lib.lib().ddf_hip_forward
                tail = (n, c, h, w, k, d, s, _lib.COMBINE[combine], _lib.DTYPE[feat.dtype],
                        _lib.VARIANT[''], ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
                calls = [tuple(ctypes.c_void_p(t.data_ptr()) for t in group) + tail for group in sets]
                for i in range(min(3, copies)):
                    _lib.check(launch(*calls[i]))
                start = torch.cuda.Event(enable_timing=True)
                stop = torch.cuda.Event(enable_timing=True)
                torch.cuda.synchronize()
                start.record()
                for i in range(iters):
                    launch(*calls[i % copies])
                stop.record()
                torch.cuda.synchronize()
            ms = start.elapsed_time(stop) / iters
            out.append({'shape': [n, c, h, w], 'stride': s, 'ms': round(ms, 4), 'bytes': nbytes,
                        'buffer_sets': copies,
                        'gbps': round(nbytes / (ms * 1e-3) / 1e9, 1),
                        'pct_of_hbm_peak': round(nbytes / (ms * 1e-3) / 8e12 * 100, 1)})
            del sets
    torch.cuda.empty_cache()
    return out
