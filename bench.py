#!/usr/bin/env python3
"""Benchmark of the DDF operator (forward + backward) on one MI355X.

A step is one forward pass plus one backward pass (all three gradients) of the
operator over one batch of synthetic input, called through the C ABI of
``libddf_hip.so`` exactly as the autograd wrapper calls it.  The default
workload is the ResNet-50 stage-3 shape the headline metric is quoted on:
N=64, C=256, 14x14, k=3 d=1 s=1, 'mul', fp32, filters standardised per tap set.

Timing: W warm-up steps, then exactly K steps between two events on the launch
stream, bracketed by device synchronisation.  Inputs and outputs rotate over
enough distinct buffer sets to exceed the 256 MB last-level cache, so the
figure is an HBM figure.  ``value`` = algorithmic bytes of forward+backward /
time per step.  Four more blocks of K steps follow; ``ms_per_step_median`` is
the median of the five.

After the timed region each library call of a step (forward / backward / the
two halves of the backward requested separately) is timed on its own: five
blocks of K back-to-back launches, median reported, same buffers.  The
``roofline`` object describes the slower call of the step; its ``traffic`` is
looked up in ``profiles/`` (hardware counters of the same kernels) and is null
when no profile covers the kernels the library reports for that call.

The same line carries the other benchmark configurations
(``other_workloads``: the fp16 'add' stage-1 shape, the strided and the
dilated 5x5 shapes, two more ResNet stages), ddf_mul_resnet50 inference
(``model_inference``: fp16, batch 128, 224x224, random weights: images/s and
per-layer GB/s of the DDF layers, operands rotating beyond the last-level
cache; ``filter_branches``: the two branch launches of DDFPack at those layers,
with and without the pooling on the spatial branch's launch), a DDFPack layer
as a training unit (``ddfpack_train``), the fused up-sampling forward
(``up_forward``), the reference's own micro-benchmark table (``test_time``) and
the CPU baseline; ``--only-headline`` leaves all but the last out.

Prints ONE JSON line on stdout; everything else goes to stderr.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E, vendor peak
LLC_BYTES = 256 * 1024 * 1024   # Infinity Cache

# name: (N, C, H, W, k, d, s, combine, dtype)
WORKLOADS = {
    'r50_stage3_mul_fp32': (64, 256, 14, 14, 3, 1, 1, 'mul', torch.float32),
    'r50_stage1_add_fp16': (64, 64, 56, 56, 3, 1, 1, 'add', torch.float16),
    'stride2_mul_fp32': (32, 128, 56, 56, 3, 1, 2, 'mul', torch.float32),
    'k5_dil2_mul_fp32': (32, 128, 56, 56, 5, 2, 1, 'mul', torch.float32),
    'r50_stage2_mul_fp32': (64, 128, 28, 28, 3, 1, 1, 'mul', torch.float32),
    'r50_stage4_mul_fp32': (64, 512, 7, 7, 3, 1, 1, 'mul', torch.float32),
}
DEFAULT_WORKLOAD = 'r50_stage3_mul_fp32'
DTYPE_NAME = {torch.float32: 'f32', torch.float16: 'f16', torch.float64: 'f64'}
# Library calls timed on their own, back to back.  The step is fwd + bwd; dx
# and dfilters are the two halves of the backward pass requested separately
# (autograd does that when only some inputs need gradients).
PHASES = ('fwd', 'bwd', 'dx', 'dfilters')
STEP_PHASES = ('fwd', 'bwd')

def log(*a):
    print(*a, file=sys.stderr, flush=True)


def standardize(f, dim):
    f = f - f.mean(dim=dim, keepdim=True)
    return f / (f.std(dim=dim, keepdim=True) + 1e-10)


def make_inputs(N, C, H, W, k, s, dtype, seed=0):
    """features, channel filter, spatial filter, grad-output ~ N(0,1) from the
    CPU generator in that order; each filter standardised over its taps."""
    g = torch.Generator(device='cpu').manual_seed(seed)
    Ho, Wo = H // s, W // s
    x = torch.randn(N, C, H, W, generator=g)
    cf = torch.randn(N, C, k, k, generator=g)
    sf = torch.randn(N, k * k, Ho, Wo, generator=g)
    go = torch.randn(N, C, Ho, Wo, generator=g)
    cf = standardize(cf.reshape(N, C, k * k), 2).reshape(N, C, k, k)
    sf = standardize(sf, 1)
    return tuple(t.to(dtype).contiguous() for t in (x, cf, sf, go))


def algorithmic_bytes(N, C, H, W, k, s, esz):
    """Every tensor touched once."""
    Ho, Wo = H // s, W // s
    X, O, CF, SF = N * C * H * W, N * C * Ho * Wo, N * C * k * k, N * k * k * Ho * Wo
    return {
        'fwd': esz * (X + O + CF + SF),
        'bwd': esz * (2 * X + O + 2 * CF + 2 * SF),
        # per library call of the backward pass
        'dx': esz * (O + CF + SF + X),
        'dfilters': esz * (O + X + CF + SF + CF + SF),
    }


def rotating_sets(N, C, H, W, k, s, esz, set_bytes):
    """Buffer sets to rotate over: enough that even the library call that touches the
    fewest bytes of a set (the forward pass) goes through twice the last-level cache
    before it sees a set again.  Sized by the whole set instead, a call timed on its own
    finds part of its operands still cached: the 5x5 forward pass then reads 30 us where
    the same kernel takes 38 us inside a step (kernel trace of both)."""
    least = min(algorithmic_bytes(N, C, H, W, k, s, esz).values())
    nsets = max(2, LLC_BYTES * 2 // least + 1)
    free, _ = torch.cuda.mem_get_info()
    return int(min(nsets, max(2, (free // 2) // set_bytes)))


class Workset(object):
    """One rotating set of device buffers for a workload."""

    def __init__(self, host):
        x, cf, sf, go = host
        self.x, self.cf, self.sf, self.go = (t.cuda() for t in (x, cf, sf, go))
        self.out = torch.empty_like(self.go)
        self.dx = torch.empty_like(self.x)
        self.dcf = torch.empty_like(self.cf)
        self.dsf = torch.empty_like(self.sf)

    def nbytes(self):
        return sum(t.numel() * t.element_size() for t in
                   (self.x, self.cf, self.sf, self.go, self.out, self.dx, self.dcf, self.dsf))


class Launcher(object):
    """Pre-built argument lists for the C ABI, so that the timed loops spend
    their host time in ``ddf_hip_forward`` / ``ddf_hip_backward`` and not in
    building ctypes objects."""

    def __init__(self, lib, sets, shape, k, d, s, combine, dtype, ws):
        N, C, H, W = shape
        self.clib = lib.lib()
        self.check = lib.check
        p = lambda t: ctypes.c_void_p(t.data_ptr())
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        tail = (N, C, H, W, k, d, s, lib.COMBINE[combine], lib.DTYPE[dtype])
        ws_bytes = ws.numel() if ws is not None else 0
        self.fwd_args = [(p(b.x), p(b.cf), p(b.sf), p(b.out)) + tail + (0, stream) for b in sets]
        self.bwd_args = {
            need: [(p(b.go), p(b.x), p(b.cf), p(b.sf), p(b.dx), p(b.dcf), p(b.dsf),
                    p(ws) if ws is not None else None, ws_bytes) + tail + (need, 0, stream)
                   for b in sets]
            for need in (lib.NEED_DX, lib.NEED_DCF | lib.NEED_DSF, 7)}
        self.n = len(sets)

    def fwd(self, i):
        rc = self.clib.ddf_hip_forward(*self.fwd_args[i % self.n])
        if rc:
            self.check(rc)

    def bwd(self, i, need=7):
        rc = self.clib.ddf_hip_backward(*self.bwd_args[need][i % self.n])
        if rc:
            self.check(rc)

    def phase(self, name, i):
        if name == 'fwd':
            self.fwd(i)
        elif name == 'bwd':
            self.bwd(i, 7)
        elif name == 'dx':
            self.bwd(i, 1)
        else:
            self.bwd(i, 6)


def timed(fn, count):
    """Milliseconds per call of fn(i), i < count, between two stream events."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for i in range(count):
        fn(i)
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / count


def timed_blocks(fn, count, blocks=5):
    """`blocks` timed blocks of `count` calls each; (first, median) in ms per call."""
    t = [timed(fn, count) for _ in range(blocks)]
    return t[0], sorted(t)[len(t) // 2]


def profiled_traffic(workload, phase, kernels):
    """HBM bytes per call from hardware counters, as recorded in profiles/*.md
    by lines of the form
        TRAFFIC workload=<name> phase=<fwd|bwd|dx|dfilters> kernels="<names>" bytes=<n>
    (FETCH_SIZE and WRITE_SIZE runs of rocprofv3, scaled as the file says).
    Returns (bytes, file name), or (None, None) when no line matches the kernels
    the library reports for this call."""
    import glob
    import re
    pat = re.compile(r'TRAFFIC workload=(\S+) phase=(\S+) kernels="([^"]*)" bytes=(\d+)')
    for path in sorted(glob.glob(os.path.join(ROOT, 'profiles', '*.md'))):
        try:
            text = open(path).read()
        except OSError:
            continue
        for m in pat.finditer(text):
            if m.group(1) == workload and m.group(2) == phase and m.group(3) == kernels:
                return int(m.group(4)), os.path.relpath(path, ROOT)
    return None, None


def profiled_kernel_us(workload, phase, kernels):
    """Sum of the traced durations of the kernels of one library call, as recorded in
    profiles/*.md by lines of the form
        KERNELTIME workload=<name> phase=<fwd|bwd> kernels="<names>" us=<microseconds>
    (rocprofv3 --kernel-trace --stats of the same call: average duration of each
    kernel times its launches per call).  Returns (us, file name) or (None, None)."""
    import glob
    import re
    pat = re.compile(r'KERNELTIME workload=(\S+) phase=(\S+) kernels="([^"]*)" us=([0-9.]+)')
    for path in sorted(glob.glob(os.path.join(ROOT, 'profiles', '*.md'))):
        try:
            text = open(path).read()
        except OSError:
            continue
        for m in pat.finditer(text):
            if m.group(1) == workload and m.group(2) == phase and m.group(3) == kernels:
                return float(m.group(4)), os.path.relpath(path, ROOT)
    return None, None


def run_workload(name, steps, warmup, lib, verbose=True, copy_probe=False):
    N, C, H, W, k, d, s, combine, dtype = WORKLOADS[name]
    esz = torch.empty(0, dtype=dtype).element_size()
    host = make_inputs(N, C, H, W, k, s, dtype)
    first = Workset(host)
    nsets = rotating_sets(N, C, H, W, k, s, esz, first.nbytes())
    sets = [first] + [Workset(host) for _ in range(nsets - 1)]
    ws_bytes = lib.backward_workspace_bytes((N, C, H, W), k, d, s, combine, dtype, 7)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device='cuda') if ws_bytes else None
    run = Launcher(lib, sets, (N, C, H, W), k, d, s, combine, dtype, ws)

    def step(i):
        run.fwd(i)
        run.bwd(i)

    for i in range(warmup):
        step(i)
    ms_per_step, ms_median = timed_blocks(step, steps)

    # each library call on its own: back-to-back launches, same buffers
    phase_ms = {}
    for ph in PHASES:
        for i in range(min(warmup, 10)):
            run.phase(ph, i)
        phase_ms[ph] = timed_blocks(lambda i, ph=ph: run.phase(ph, i), steps)[1]
    need_of = {'fwd': 0, 'bwd': 7, 'dx': 1, 'dfilters': 6}
    kernels = {ph: lib.describe((N, C, H, W), k, d, s, combine, dtype, need_of[ph]) for ph in PHASES}

    if copy_probe:
        # a plain device copy of known size: the yardstick the hardware
        # fetch/write counters are scaled by
        a = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device='cuda')
        b = torch.empty_like(a)
        for _ in range(4):
            b.copy_(a)
        torch.cuda.synchronize()

    ab = algorithmic_bytes(N, C, H, W, k, s, esz)
    total = ab['fwd'] + ab['bwd']
    res = {
        'workload': name, 'N': N, 'C': C, 'H': H, 'W': W, 'k': k, 'd': d, 's': s,
        'combine': combine, 'dtype': DTYPE_NAME[dtype],
        'ms_per_step': ms_per_step, 'ms_per_step_median': ms_median, 'kernels': kernels,
        'gbps': total / (ms_per_step * 1e-3) / 1e9,
        'images_per_s': N / (ms_per_step * 1e-3),
        'bytes': ab, 'phase_ms': phase_ms, 'buffer_sets': nsets,
        'phase_gbps': {p: ab[p] / (phase_ms[p] * 1e-3) / 1e9 for p in PHASES},
    }
    if verbose:
        log('[%s] %.1f us/step  fwd+bwd %.0f GB/s (%.1f%% of HBM peak), %d buffer sets' % (
            name, ms_per_step * 1e3, res['gbps'], 100 * res['gbps'] / HBM_PEAK_GBPS, nsets))
        for p in PHASES:
            log('    %-9s %7.1f us  %6.0f GB/s  %.1f%%' % (
                p, phase_ms[p] * 1e3, res['phase_gbps'][p],
                100 * res['phase_gbps'][p] / HBM_PEAK_GBPS))
    del sets, first, run
    torch.cuda.empty_cache()
    return res


def profile_phase(name, phase, steps, warmup, lib):
    """One library call of a workload on its own, for runs under rocprofv3:
    warmup + steps calls of `phase` over the rotating buffer sets, then a plain
    256 MiB device copy (the yardstick the fetch / write counters are scaled by).
    Every ddf:: dispatch of the process belongs to that call."""
    N, C, H, W, k, d, s, combine, dtype = WORKLOADS[name]
    host = make_inputs(N, C, H, W, k, s, dtype)
    first = Workset(host)
    esz = torch.empty(0, dtype=dtype).element_size()
    nsets = rotating_sets(N, C, H, W, k, s, esz, first.nbytes())
    sets = [first] + [Workset(host) for _ in range(nsets - 1)]
    ws_bytes = lib.backward_workspace_bytes((N, C, H, W), k, d, s, combine, dtype, 7)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device='cuda') if ws_bytes else None
    run = Launcher(lib, sets, (N, C, H, W), k, d, s, combine, dtype, ws)
    for i in range(warmup):
        run.phase(phase, i)
    ms = timed(lambda i: run.phase(phase, i), steps)
    a = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device='cuda')
    b = torch.empty_like(a)
    for _ in range(4):
        b.copy_(a)
    torch.cuda.synchronize()
    need_of = {'fwd': 0, 'bwd': 7, 'dx': 1, 'dfilters': 6}
    return {'workload': name, 'phase': phase, 'calls': warmup + steps, 'us_per_call': round(ms * 1e3, 2),
            'kernels': lib.describe((N, C, H, W), k, d, s, combine, dtype, need_of[phase]),
            'algorithmic_bytes': algorithmic_bytes(N, C, H, W, k, s, esz)[phase],
            'copy_probe_bytes': 4 * a.numel() * 4}


BRANCH_LAYERS = ((64, 56, 1, 3), (128, 56, 2, 1), (128, 28, 1, 3), (256, 28, 2, 1), (256, 14, 1, 5),
                 (512, 14, 2, 1), (512, 7, 1, 2))   # (C, H = W, stride, layers of that shape in ddf_mul_resnet50)


def profile_branch(index, which, steps, warmup, lib, batch=128):
    """One filter-branch launch shape on its own, for runs under rocprofv3:
    warmup + steps launches of the spatial (or channel) branch kernel at layer
    shape BRANCH_LAYERS[index], fp16, feature maps rotating beyond the
    last-level cache, then a plain 256 MiB device copy (the yardstick the fetch /
    write counters are scaled by)."""
    dt = torch.float16
    c, hw, s, count = BRANCH_LAYERS[index]
    mid = int(c * 0.2)
    torch.manual_seed(0)
    nset = max(2, int(600e6 / (batch * c * hw * hw * 2)) + 1)
    if which in ('spatial', 'spatial_pool'):
        w = torch.randn(9, c, device='cuda', dtype=dt) * 0.1
        b = torch.randn(9, device='cuda', dtype=dt)
        xs = [torch.randn(batch, c, hw, hw, device='cuda', dtype=dt) for _ in range(nset)]
        call = lib.spatial_branch if which == 'spatial' else lib.spatial_branch_pool
        run = lambda i: call(xs[i % nset], w, b, 1, 3, s, 1.0, None, None)
        # (what the branch needs; the pooled variant needs every row under stride 2 as well)
        nbytes = batch * c * hw * hw * 2 // (s if which == 'spatial' else 1) + batch * 9 * (hw // s) ** 2 * 2
    else:
        w1 = torch.randn(mid, c, device='cuda', dtype=dt) * 0.1
        b1 = torch.randn(mid, device='cuda', dtype=dt)
        w2 = torch.randn(c * 9, mid, device='cuda', dtype=dt) * 0.1
        b2 = torch.randn(c * 9, device='cuda', dtype=dt)
        gv = torch.ones(c * 9, device='cuda', dtype=dt)
        ov = torch.zeros(c * 9, device='cuda', dtype=dt)
        ps = [torch.randn(batch, c, device='cuda', dtype=dt) for _ in range(nset)]
        run = lambda i: lib.channel_branch(ps[i % nset], w1, b1, w2, b2, 3, 1.0, gv, ov)
        nbytes = 2 * (batch * c + mid * c + c * 9 * mid + batch * c * 9)
    for i in range(warmup):
        run(i)
    ms = timed(run, steps)
    a = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device='cuda')
    b_ = torch.empty_like(a)
    for _ in range(4):
        b_.copy_(a)
    torch.cuda.synchronize()
    return {'branch': which, 'shape': [batch, c, hw, hw], 'stride': s, 'layers': count,
            'calls': warmup + steps, 'us_per_call': round(ms * 1e3, 2), 'algorithmic_bytes': nbytes,
            'copy_probe_bytes': 4 * a.numel() * 4}


def device_copy_ceiling(step_bytes):
    """What a plain device-to-device copy reaches on this box: the practical
    ceiling beside the 8 TB/s of the data sheet.  Once at 256 MiB, once moving as
    many bytes as one forward call of the workload (read half, write half),
    rotating over enough buffers to stay out of the last-level cache."""
    big_a = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device='cuda')
    big_b = torch.empty_like(big_a)
    for _ in range(3):
        big_b.copy_(big_a)
    ms_big = timed(lambda i: big_b.copy_(big_a), 10)
    big_bytes = 2 * big_a.numel() * 4
    del big_a, big_b
    half = max(1, step_bytes // 8)             # floats per side
    pairs = int(max(2, 2 * LLC_BYTES // (half * 8) + 1))
    src = [torch.empty(half, dtype=torch.float32, device='cuda') for _ in range(pairs)]
    dst = [torch.empty(half, dtype=torch.float32, device='cuda') for _ in range(pairs)]
    for i in range(pairs):
        dst[i].copy_(src[i])
    ms_small = timed(lambda i: dst[i % pairs].copy_(src[i % pairs]), 100)
    out = {'bytes_large': big_bytes, 'gbps_large': round(big_bytes / (ms_big * 1e-3) / 1e9, 1),
           'bytes_small': half * 8, 'us_small': round(ms_small * 1e3, 2),
           'gbps_small': round(half * 8 / (ms_small * 1e-3) / 1e9, 1)}
    del src, dst
    torch.cuda.empty_cache()
    return out


def profile_model(batches=5, warmup=4, batch=128):
    """ddf_mul_resnet50 fp16 inference for runs under rocprofv3: warm-up batches (in which
    the convolution library searches its kernels), half a second of silence, then `batches`
    timed batches - the dispatches after the gap in the trace are the steady state."""
    import time
    from ddfnet_amd import ddf_resnet
    torch.manual_seed(0)
    model = ddf_resnet.ddf_mul_resnet50(zero_init_last_bn=False).cuda().half().eval()
    x = torch.randn(batch, 3, 224, 224, device='cuda', dtype=torch.float16)
    with torch.no_grad():
        for _ in range(warmup):
            model(x)
        torch.cuda.synchronize()
        time.sleep(0.5)
        ms = timed(lambda i: model(x), batches)
    return {'model': 'ddf_mul_resnet50', 'batch': batch, 'dtype': 'f16', 'batches': batches,
            'ms_per_batch': round(ms, 3)}


def cpu_baseline(name, budget_s=12.0):
    """The CPU oracle (a port of the reference's formulation; the reference has
    no CPU path of its own) timed on this host: fp32, forward + backward, on a
    the whole batch of the workload,
    repeated until the time budget is used."""
    import oracle
    N, C, H, W, k, d, s, combine, dtype = WORKLOADS[name]
    n_sub = N
    x, cf, sf, go = (t.float() for t in make_inputs(n_sub, C, H, W, k, s, dtype))
    threads = oracle.num_threads()

    def once():
        oracle.forward_f32(x, cf, sf, k, d, s, combine)
        oracle.backward_f32(go, x, cf, sf, k, d, s, combine)

    once()
    t0 = time.perf_counter()
    reps = 0
    while True:
        once()
        reps += 1
        el = time.perf_counter() - t0
        if el > budget_s:
            break
    per = el / reps
    ab = algorithmic_bytes(n_sub, C, H, W, k, s, 4)
    return {
        'value': round((ab['fwd'] + ab['bwd']) / per / 1e9, 3), 'unit': 'GB/s',
        'cores': threads, 'kind': 'port',
        'sample': 'all %d samples of %s in fp32, forward+backward, %d repetitions in %.1f s '
                  '(%.4f s each), C oracle with OpenMP' % (N, name, reps, el, per),
        'images_per_s': round(n_sub / per, 1),
    }


def model_inference(batch=128, steps=10, warmup=3):
    """ddf_mul_resnet50 inference, fp16, random weights, synthetic input."""
    from ddfnet_amd import ddf_resnet
    torch.manual_seed(0)
    model = ddf_resnet.ddf_mul_resnet50(zero_init_last_bn=False).cuda().half().eval()
    x = torch.randn(batch, 3, 224, 224, device='cuda', dtype=torch.float16)
    with torch.no_grad():
        for _ in range(warmup):
            model(x)
        ms = timed_blocks(lambda i: model(x), steps)[1]
        layers = ddf_resnet.time_ddf_layers(model, x)
        # the same network with the BatchNorms that follow convolutions folded into them
        folded = ddf_resnet.fold_batchnorm(model)
        for _ in range(warmup):
            folded(x)
        ms_folded = timed_blocks(lambda i: folded(x), steps)[1]
        del folded
    ddf_ms = sum(l['ms'] for l in layers)
    ddf_bytes = sum(l['bytes'] for l in layers)
    return {'model': 'ddf_mul_resnet50', 'batch': batch, 'dtype': 'f16', 'input': [batch, 3, 224, 224],
            'weights': 'random (Kaiming normal, BatchNorm at default init)',
            'images_per_s': round(batch / (ms * 1e-3), 1), 'ms_per_batch': round(ms, 3),
            'images_per_s_folded_batchnorm': round(batch / (ms_folded * 1e-3), 1),
            'ms_per_batch_folded_batchnorm': round(ms_folded, 3),
            'ddf_ms_per_batch': round(ddf_ms, 3),
            'ddf_gbps': round(ddf_bytes / (ddf_ms * 1e-3) / 1e9, 1) if ddf_ms else None,
            'ddf_layers': layers}


def branch_table(lib, batch=128, iters=100):
    """The two filter-branch launches of DDFPack at the sixteen DDF layers of
    ddf_mul_resnet50 (ddf/ddf.py:176-192, inference, fp16), each timed on its
    own between stream events with feature maps rotating beyond the last-level
    cache, and torch's global average pool over the same feature maps; then the
    pair the module runs instead, with the pooling on the spatial branch's launch.
    GB/s: feature bytes the spatial branch must read (every second row under
    stride 2) plus the taps it writes."""
    dt = torch.float16
    layers = BRANCH_LAYERS

    def timed(fns):
        n = len(fns)
        for i in range(n + 3):
            fns[i % n]()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record()
        for i in range(iters):
            fns[i % n]()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / iters * 1e3

    rows, total = [], {'spatial_us': 0.0, 'channel_us': 0.0, 'pool_us': 0.0, 'spatial_with_pool_us': 0.0,
                       'channel_from_parts_us': 0.0}
    torch.manual_seed(0)
    for c, hw, s, count in layers:
        mid = int(c * 0.2)
        nset = max(2, int(600e6 / (batch * c * hw * hw * 2)) + 1)
        w1 = torch.randn(mid, c, device='cuda', dtype=dt) * 0.1
        b1 = torch.randn(mid, device='cuda', dtype=dt)
        w2 = torch.randn(c * 9, mid, device='cuda', dtype=dt) * 0.1
        b2 = torch.randn(c * 9, device='cuda', dtype=dt)
        gv = torch.ones(c * 9, device='cuda', dtype=dt)
        ov = torch.zeros(c * 9, device='cuda', dtype=dt)
        w = torch.randn(9, c, device='cuda', dtype=dt) * 0.1
        b = torch.randn(9, device='cuda', dtype=dt)
        xs = [torch.randn(batch, c, hw, hw, device='cuda', dtype=dt) for _ in range(nset)]
        ps = [torch.randn(batch, c, device='cuda', dtype=dt) for _ in range(nset)]
        ch = timed([(lambda q=q: lib.channel_branch(q, w1, b1, w2, b2, 3, 1.0, gv, ov)) for q in ps])
        sp = timed([(lambda x=x: lib.spatial_branch(x, w, b, 1, 3, s, 1.0, None, None)) for x in xs])
        pool = timed([(lambda x=x: x.mean((2, 3))) for x in xs])
        # the same with the pooling riding on the spatial branch's launch
        sp_pool = timed([(lambda x=x: lib.spatial_branch_pool(x, w, b, 1, 3, s, 1.0, None, None)) for x in xs])
        parts = [lib.spatial_branch_pool(x, w, b, 1, 3, s, 1.0, None, None)[1] for x in xs[:2]]
        ch_parts = timed([(lambda q=q: lib.channel_branch_parts(q, 1.0 / (hw * hw), w1, b1, w2, b2, 3, 1.0, gv, ov))
                          for q in parts])
        nbytes = batch * c * hw * hw * 2 // s + batch * 9 * (hw // s) ** 2 * 2
        rows.append({'shape': [batch, c, hw, hw], 'stride': s, 'layers': count,
                     'spatial_us': round(sp, 1), 'spatial_gbps': round(nbytes / sp / 1e3, 1),
                     'channel_us': round(ch, 1), 'torch_mean_us': round(pool, 1),
                     'spatial_with_pool_us': round(sp_pool, 1), 'channel_from_parts_us': round(ch_parts, 1)})
        total['spatial_us'] += count * sp
        total['channel_us'] += count * ch
        total['pool_us'] += count * pool
        total['spatial_with_pool_us'] += count * sp_pool
        total['channel_from_parts_us'] += count * ch_parts
        del xs, parts
    torch.cuda.empty_cache()
    out = {'per_batch_of_%d' % batch: {k: round(v, 1) for k, v in total.items()}, 'layers': rows}
    log('[branches] per batch of %d, 16 layers: pool %.0f + channel %.0f + spatial %.0f = %.0f us; with the pooling '
        'on the spatial launch: channel %.0f + spatial %.0f = %.0f us' % (
            batch, total['pool_us'], total['channel_us'], total['spatial_us'],
            total['pool_us'] + total['channel_us'] + total['spatial_us'],
            total['channel_from_parts_us'], total['spatial_with_pool_us'],
            total['channel_from_parts_us'] + total['spatial_with_pool_us']))
    return out


def test_time_table(iters=20, warmup=5):
    """The reference's own micro-benchmark (test_time.py:54-145): a 3x3
    convolution, a depthwise 3x3 convolution, a DDFPack layer and the bare ddf
    operator ('mul', k=3) on fp32 feature maps of 256 channels, inference only.
    Times are per call in milliseconds, between stream events."""
    import torch.nn as nn
    from ddfnet_amd import DDFPack, ddf
    shapes = [(2, 200, 300), (32, 224, 224), (32, 112, 112), (32, 56, 56), (32, 28, 28),
              (32, 14, 14), (32, 7, 7)]
    torch.manual_seed(0)
    conv = nn.Conv2d(256, 256, 3, padding=1).cuda().eval()
    dw_conv = nn.Conv2d(256, 256, 3, padding=1, groups=256).cuda().eval()
    layer = DDFPack(256).cuda().eval()
    rows = []
    with torch.no_grad():
        for n, h, w in shapes:
            feat = torch.randn(n, 256, h, w, device='cuda')
            spatial = torch.rand(n, 9, h, w, device='cuda')
            channel = torch.rand(n, 256, 3, 3, device='cuda')
            row = {'shape': [n, 256, h, w]}
            for name, fn in (('conv', lambda: conv(feat)), ('dw_conv', lambda: dw_conv(feat)),
                             ('ddf_layer', lambda: layer(feat)),
                             ('ddf_op', lambda: ddf(feat, channel, spatial, 3, 1, 1, 'mul'))):
                for _ in range(warmup):
                    fn()
                row[name + '_ms'] = round(timed(lambda i: fn(), iters), 4)
            ab = algorithmic_bytes(n, 256, h, w, 3, 1, 4)['fwd']
            row['ddf_op_gbps'] = round(ab / (row['ddf_op_ms'] * 1e-3) / 1e9, 1)
            rows.append(row)
            log('[test_time] %s conv %.3f  dw_conv %.3f  ddf_layer %.3f  ddf_op %.3f ms (%.0f GB/s)' % (
                row['shape'], row['conv_ms'], row['dw_conv_ms'], row['ddf_layer_ms'],
                row['ddf_op_ms'], row['ddf_op_gbps']))
            del feat, spatial, channel
            torch.cuda.empty_cache()
    return rows


def pack_train_table(iters=30, warmup=8):
    """DDFPack (ddf/ddf.py:195-222) as a training unit: forward + backward (input and
    parameter gradients) of one layer at the three stride-1 ResNet-50 stage shapes, fp32
    and fp16.  `fused`: the spatial filter normalisation and the operator as one autograd
    node whose backward pushes dSF through the normalisation inside the partial-sum
    launch (the default); `op_by_op`: the normalisation as a module of its own in front
    of the operator, as in the reference.  A step is host-bound at these sizes (about
    thirty launches issued from Python), so beside the time per step the table gives the
    launches per step and the summed durations of their kernels, both from torch's
    profiler (null where that is not available)."""
    from ddfnet_amd import DDFPack
    shapes = [(64, 64, 56, 56), (64, 128, 28, 28), (64, 256, 14, 14)]
    rows = []

    def launches(step):
        """(kernel launches, summed kernel durations in us) of one step."""
        try:
            from torch.profiler import profile, ProfilerActivity
            with profile(activities=[ProfilerActivity.CUDA]) as prof:
                step()
                torch.cuda.synchronize()
            kernels = [e for e in prof.events() if getattr(e, 'device_type', None) is not None and
                       str(e.device_type).endswith('CUDA')]
            return len(kernels), round(sum(e.time_range.elapsed_us() for e in kernels), 1)
        except Exception:    # profiler back end missing on this box
            return None, None

    for dtype in (torch.float32, torch.float16):
        for n, c, h, w in shapes:
            torch.manual_seed(0)
            layer = DDFPack(c).cuda().to(dtype).train()
            x = torch.randn(n, c, h, w, device='cuda').to(dtype).requires_grad_(True)
            go = torch.randn(n, c, h, w, device='cuda').to(dtype)
            row = {'shape': [n, c, h, w], 'dtype': DTYPE_NAME[dtype]}
            for name, fused in (('fused', True), ('op_by_op', False)):
                layer.fuse_spatial_norm = fused

                def step():
                    layer.zero_grad(set_to_none=True)
                    x.grad = None
                    layer(x).backward(go)

                for _ in range(warmup):
                    step()
                row[name + '_us'] = round(timed(lambda i: step(), iters) * 1e3, 1)
                row[name + '_launches'], row[name + '_kernel_us'] = launches(step)
            rows.append(row)
            log('[pack-train] DDFPack(%d) %s %s: fused %.1f us per step (%s launches, %s us of kernels), '
                'op by op %.1f us (%s launches, %s us of kernels)' % (
                    c, row['shape'], row['dtype'], row['fused_us'], row['fused_launches'],
                    row['fused_kernel_us'], row['op_by_op_us'], row['op_by_op_launches'],
                    row['op_by_op_kernel_us']))
            del layer, x, go
            torch.cuda.empty_cache()
    return rows


def up_forward_table(lib, iters=50, warmup=10):
    """The up-sampling operator of DDFUpPack (ddf/ddf.py:264-272), forward only:
    one fused launch against the reference's composition (one ddf call per
    sub-pixel branch, torch.stack, F.pixel_shuffle).  Algorithmic bytes: the
    features once, every branch's two filters once, the up-sampled result once."""
    import torch.nn.functional as F
    from ddfnet_amd import ddf
    cases = [(8, 64, 64, 64, 3, 2, torch.float32), (8, 64, 64, 64, 3, 2, torch.float16),
             (4, 64, 128, 128, 3, 2, torch.float32), (16, 128, 32, 32, 3, 2, torch.float32),
             (8, 64, 64, 64, 3, 3, torch.float32), (8, 64, 64, 64, 5, 2, torch.float32)]
    rows = []
    with torch.no_grad():
        for n, c, h, w, k, r, dtype in cases:
            x = torch.randn(n, c, h, w, device='cuda').to(dtype)
            cfs = [torch.randn(n, c, k, k, device='cuda').to(dtype) for _ in range(r * r)]
            sfs = [torch.randn(n, k * k, h, w, device='cuda').to(dtype) for _ in range(r * r)]

            def composed():
                outs = [ddf(x, cf, sf, k, 1, 1, 'mul') for cf, sf in zip(cfs, sfs)]
                return F.pixel_shuffle(torch.stack(outs, dim=2).reshape(n, -1, h, w), r)

            out = torch.empty(n, c, h * r, w * r, device='cuda', dtype=dtype)
            cf_ptrs = (ctypes.c_void_p * (r * r))(*[t.data_ptr() for t in cfs])
            sf_ptrs = (ctypes.c_void_p * (r * r))(*[t.data_ptr() for t in sfs])
            stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            entry = lib.lib().ddf_hip_up_forward

            def fused():   # the C entry point, as the other figures of this file
                rc = entry(x.data_ptr(), cf_ptrs, sf_ptrs, out.data_ptr(), n, c, h, w, k, 1, r,
                           0, lib.DTYPE[dtype], stream)
                assert rc == 0

            esz = x.element_size()
            nbytes = esz * (x.numel() * (1 + r * r) + sum(t.numel() for t in cfs + sfs))
            row = {'shape': [n, c, h, w], 'k': k, 'scale': r, 'dtype': DTYPE_NAME[dtype],
                   'bytes': nbytes}
            for name, fn in (('fused', fused), ('composed', composed)):
                for _ in range(warmup):
                    fn()
                row[name + '_us'] = round(timed(lambda i: fn(), iters) * 1e3, 2)
            row['fused_gbps'] = round(nbytes / (row['fused_us'] * 1e-6) / 1e9, 1)
            row['speedup'] = round(row['composed_us'] / row['fused_us'], 2)
            rows.append(row)
            log('[up] %s k%d x%d %s: fused %.1f us (%.0f GB/s, %.1f%% of HBM peak)  composed %.1f us  x%.2f' % (
                row['shape'], k, r, row['dtype'], row['fused_us'], row['fused_gbps'],
                100 * row['fused_gbps'] / HBM_PEAK_GBPS, row['composed_us'], row['speedup']))
    return rows


def roofline_of(res):
    """Roofline object of a workload: the slower call of its step (forward or
    backward), algorithmic bytes of that call / its median launch time."""
    dominant = max(STEP_PHASES, key=lambda p: res['phase_ms'][p])
    nbytes = res['bytes'][dominant]
    sec = res['phase_ms'][dominant] * 1e-3
    achieved = nbytes / sec / 1e9
    traffic, source = profiled_traffic(res['workload'], dominant, res['kernels'][dominant])
    out = {'bound': 'hbm', 'phase': dominant, 'kernel': res['kernels'][dominant],
           'achieved': round(achieved, 2), 'peak': HBM_PEAK_GBPS, 'unit': 'GB/s',
           'frac': round(achieved / HBM_PEAK_GBPS, 4), 'traffic': traffic,
           'traffic_source': source, 'bytes_per_launch': nbytes,
           'avg_launch_us': round(sec * 1e6, 3)}
    # The same fraction from the committed kernel trace: algorithmic bytes / summed traced
    # kernel durations.  It is lower than `frac` where a call is several kernels: the
    # trace adds their durations up, while on the stream the next kernel's start
    # overlaps the previous one's drain, which the events around the call see.
    prof_us, prof_src = profiled_kernel_us(res['workload'], dominant, res['kernels'][dominant])
    if prof_us:
        out['profile_kernel_us'] = prof_us
        out['frac_from_profile'] = round(nbytes / (prof_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)
        out['profile_source'] = prof_src
        out['frac_note'] = ('frac: events around back-to-back calls in this run; frac_from_profile: '
                            'summed kernel durations of the committed rocprofv3 trace')
    return out


def workload_summary(r):
    """What the JSON line carries for a workload other than the headline one."""
    return {
        'config': '%s: N=%d C=%d H=W=%d k=%d d=%d s=%d %s %s' % (
            r['workload'], r['N'], r['C'], r['H'], r['k'], r['d'], r['s'], r['combine'], r['dtype']),
        'gbps': round(r['gbps'], 1), 'pct_of_hbm_peak': round(100 * r['gbps'] / HBM_PEAK_GBPS, 2),
        'us_per_step': round(r['ms_per_step'] * 1e3, 2),
        'us_per_step_median': round(r['ms_per_step_median'] * 1e3, 2),
        'images_per_s': round(r['images_per_s'], 1),
        'bytes_per_step': r['bytes']['fwd'] + r['bytes']['bwd'],
        'phases_us': {p: round(r['phase_ms'][p] * 1e3, 2) for p in PHASES},
        'phases_pct_of_hbm_peak': {p: round(100 * r['phase_gbps'][p] / HBM_PEAK_GBPS, 1) for p in PHASES},
        'kernels': r['kernels'], 'roofline': roofline_of(r)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=100)
    ap.add_argument('--warmup', type=int, default=20)
    ap.add_argument('--workload', default=DEFAULT_WORKLOAD, choices=sorted(WORKLOADS))
    ap.add_argument('--only-headline', action='store_true',
                    help='time the headline workload only (no other workloads, no model)')
    ap.add_argument('--all', action='store_true', help='(default now; kept for old command lines)')
    ap.add_argument('--model', action='store_true', help='(default now; kept for old command lines)')
    ap.add_argument('--test-time', action='store_true',
                    help="with --only-headline: also run the reference's micro-benchmark table (conv, "
                         "depthwise conv, DDFPack, ddf at seven 256-channel shapes; part of the default "
                         "line otherwise)")
    ap.add_argument('--up-pack', action='store_true',
                    help='with --only-headline: also time the fused up-sampling forward against its '
                         'composition (part of the default line otherwise)')
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg')
    ap.add_argument('--profile-phase', choices=PHASES, default=None,
                    help='run only this library call of the workload (warm-up + steps calls, then the '
                         'copy probe) and print what was run: the unit the profiles/ summaries are '
                         'collected on')
    ap.add_argument('--profile-model', action='store_true',
                    help='run only the ResNet-50 inference (warm-up, a half-second gap, then --steps '
                         'batches): the unit the model summary in profiles/ is collected on')
    ap.add_argument('--profile-branch', default=None, metavar='KIND:INDEX',
                    help='run only the spatial or channel branch launch of one ResNet-50 layer shape '
                         '(spatial:0 .. spatial:6, spatial_pool:0 .. 6, channel:0 .. channel:6): the unit the branch summary in '
                         'profiles/ is collected on')
    ap.add_argument('--copy-probe', action='store_true',
                    help='also run a plain 256 MiB device copy (calibrates hardware counters)')
    args = ap.parse_args()
    if args.gpus != 1:
        log('bench.py measures one GPU: the operator shards over the batch with no exchange, '
            'and this build runs on a single device.  Re-run with --gpus 1.')
        sys.exit(2)
    assert torch.cuda.is_available(), 'bench.py needs a GPU'
    torch.cuda.set_device(0)
    from ddfnet_amd import _lib as lib
    lib.lib()

    if args.profile_model:
        print(json.dumps(profile_model(batches=args.steps)))
        return
    if args.profile_branch:
        kind, index = args.profile_branch.split(':')
        assert kind in ('spatial', 'spatial_pool', 'channel') and 0 <= int(index) < len(BRANCH_LAYERS)
        print(json.dumps(profile_branch(int(index), kind, args.steps, args.warmup, lib)))
        return
    if args.profile_phase:
        print(json.dumps(profile_phase(args.workload, args.profile_phase, args.steps, args.warmup, lib)))
        return
    res = run_workload(args.workload, args.steps, args.warmup, lib, copy_probe=args.copy_probe)
    extra = {}
    if not args.only_headline:
        for name in WORKLOADS:
            if name != args.workload:
                extra[name] = run_workload(name, args.steps, args.warmup, lib)

    line = {
        'metric': 'ddf_fwd_bwd_hbm_gbps', 'value': round(res['gbps'], 2), 'unit': 'GB/s',
        'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
        'ms_per_step': round(res['ms_per_step'], 6), 'higher_is_better': True,
        'scaling': 'weak', 'vs_baseline': None, 'dtype': res['dtype'], 'data': 'synthetic',
        'config': {'workload': '%s: N=%d C=%d H=W=%d k=%d d=%d s=%d %s %s' % (
            res['workload'], res['N'], res['C'], res['H'], res['k'], res['d'], res['s'],
            res['combine'], res['dtype']),
            'bytes_per_step': res['bytes']['fwd'] + res['bytes']['bwd'],
            'buffer_sets': res['buffer_sets']},
        'ms_per_step_median': round(res['ms_per_step_median'], 6),
        'pct_of_hbm_peak': round(100 * res['gbps'] / HBM_PEAK_GBPS, 2),
        'images_per_s': round(res['images_per_s'], 1),
        'roofline': roofline_of(res),
        'phases_us': {p: round(res['phase_ms'][p] * 1e3, 3) for p in PHASES},
        'kernels': res['kernels'],
    }
    if extra:
        line['other_workloads'] = {n: workload_summary(r) for n, r in extra.items()}
    line['device_copy'] = device_copy_ceiling(res['bytes']['fwd'])
    dc = line['device_copy']
    log('[copy] device-to-device copy: %.0f GB/s moving %d MiB; %.0f GB/s (%.1f us) moving the %.1f MB of a forward call' % (
        dc['gbps_large'], dc['bytes_large'] >> 20, dc['gbps_small'], dc['us_small'], dc['bytes_small'] / 1e6))
    if not args.only_headline:
        line['model_inference'] = model_inference()
        mi = line['model_inference']
        log('[model] %s bs%d %s: %.1f images/s (%.2f ms/batch, DDF layers %.2f ms)' % (
            mi['model'], mi['batch'], mi['dtype'], mi['images_per_s'], mi['ms_per_batch'],
            mi['ddf_ms_per_batch']))
    if not args.only_headline:
        line['model_inference']['filter_branches'] = branch_table(lib)
        line['ddfpack_train'] = pack_train_table()
        line['up_forward'] = up_forward_table(lib)
    elif args.up_pack:
        line['up_forward'] = up_forward_table(lib)
    if args.test_time or not args.only_headline:
        line['test_time'] = test_time_table()
    if not args.no_cpu:
        line['cpu_baseline'] = cpu_baseline(args.workload)
        cb = line['cpu_baseline']
        log('[cpu] %s: %.2f GB/s on %d threads' % (cb['sample'], cb['value'], cb['cores']))
    print(json.dumps(line), flush=True)


if __name__ == '__main__':
    main()
