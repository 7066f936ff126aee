#!/usr/bin/env python3
"""Benchmark of the DDF operator (forward + backward) on one MI355X.

A step is one forward pass plus one backward pass (all three gradients) of the
operator over one batch of synthetic input, called through the C ABI of
``libddf_hip.so`` exactly as the autograd wrapper calls it.  The default
workload is the ResNet-50 stage-3 shape the headline metric is quoted on:
N=64, C=256, 14x14, k=3 d=1 s=1, 'mul', fp32, filters standardised per tap set.

Timing: W warm-up steps, then K steps between two events on the launch stream,
bracketed by device synchronisation.  Inputs and outputs rotate over enough
distinct buffer sets to exceed the 256 MB last-level cache, so the figure is an
HBM figure.  ``value`` = algorithmic bytes of forward+backward / time per step.

After the timed region the same K steps are replayed with an event pair around
every library call (forward / feature gradient / filter gradients) to obtain the
per-kernel durations the ``roofline`` object reports for the dominant kernel.

Prints ONE JSON line on stdout; everything else goes to stderr.
"""
import argparse
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
        # per kernel of the backward pass
        'dx': esz * (O + CF + SF + X),
        'dfilters': esz * (O + X + CF + SF + CF + SF),
    }


class Workset(object):
    """One rotating set of device buffers for a workload."""

    def __init__(self, host, like=None):
        x, cf, sf, go = host
        self.x, self.cf, self.sf, self.go = (t.cuda() for t in (x, cf, sf, go))
        self.out = torch.empty_like(self.go)
        self.dx = torch.empty_like(self.x)
        self.dcf = torch.empty_like(self.cf)
        self.dsf = torch.empty_like(self.sf)

    def nbytes(self):
        return sum(t.numel() * t.element_size() for t in
                   (self.x, self.cf, self.sf, self.go, self.out, self.dx, self.dcf, self.dsf))


def run_workload(name, steps, warmup, lib, verbose=True):
    N, C, H, W, k, d, s, combine, dtype = WORKLOADS[name]
    esz = torch.empty(0, dtype=dtype).element_size()
    host = make_inputs(N, C, H, W, k, s, dtype)
    first = Workset(host)
    nsets = max(2, LLC_BYTES * 2 // first.nbytes() + 1)
    free, _ = torch.cuda.mem_get_info()
    nsets = int(min(nsets, max(2, (free // 2) // first.nbytes())))
    sets = [first] + [Workset(host) for _ in range(nsets - 1)]
    need_all = lib.NEED_DX | lib.NEED_DCF | lib.NEED_DSF
    ws_bytes = lib.backward_workspace_bytes((N, C, H, W), k, d, s, combine, dtype, need_all)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device='cuda')

    def fwd(b):
        lib.forward(b.x, b.cf, b.sf, b.out, k, d, s, combine)

    def bwd(b, need=need_all):
        lib.backward(b.go, b.x, b.cf, b.sf, b.dx, b.dcf, b.dsf, k, d, s, combine, need, ws)

    def step(i):
        b = sets[i % nsets]
        fwd(b)
        bwd(b)

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(steps):
        step(i)
    stop.record()
    torch.cuda.synchronize()
    ms_per_step = start.elapsed_time(stop) / steps

    # replay with an event pair around every library call
    phases = {'fwd': lambda b: fwd(b),
              'dx': lambda b: bwd(b, lib.NEED_DX),
              'dfilters': lambda b: bwd(b, lib.NEED_DCF | lib.NEED_DSF)}
    evs = {p: [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
               for _ in range(steps)] for p in phases}
    for i in range(steps):
        b = sets[i % nsets]
        for p, fn in phases.items():
            e0, e1 = evs[p][i]
            e0.record()
            fn(b)
            e1.record()
    torch.cuda.synchronize()
    phase_ms = {}
    for p in phases:
        ts = sorted(e0.elapsed_time(e1) for e0, e1 in evs[p])
        phase_ms[p] = {'mean': sum(ts) / len(ts), 'median': ts[len(ts) // 2], 'min': ts[0]}

    ab = algorithmic_bytes(N, C, H, W, k, s, esz)
    total = ab['fwd'] + ab['bwd']
    res = {
        'workload': name, 'N': N, 'C': C, 'H': H, 'W': W, 'k': k, 'd': d, 's': s,
        'combine': combine, 'dtype': DTYPE_NAME[dtype],
        'ms_per_step': ms_per_step,
        'gbps': total / (ms_per_step * 1e-3) / 1e9,
        'images_per_s': N / (ms_per_step * 1e-3),
        'bytes': ab, 'phase_ms': phase_ms, 'buffer_sets': nsets,
        'phase_gbps': {p: ab[p] / (phase_ms[p]['mean'] * 1e-3) / 1e9 for p in phases},
    }
    if verbose:
        log('[%s] %.1f us/step  fwd+bwd %.0f GB/s (%.1f%% of HBM peak), %d buffer sets' % (
            name, ms_per_step * 1e3, res['gbps'], 100 * res['gbps'] / HBM_PEAK_GBPS, nsets))
        for p in phases:
            log('    %-9s %7.1f us (median %.1f, min %.1f)  %6.0f GB/s  %.1f%%' % (
                p, phase_ms[p]['mean'] * 1e3, phase_ms[p]['median'] * 1e3, phase_ms[p]['min'] * 1e3,
                res['phase_gbps'][p], 100 * res['phase_gbps'][p] / HBM_PEAK_GBPS))
    del sets, first
    torch.cuda.empty_cache()
    return res


def cpu_baseline(name, budget_s=15.0):
    """The CPU oracle (a port of the reference's formulation; the reference has
    no CPU path of its own) timed on this host: fp32, forward + backward, on a
    batch slice sized to finish within the budget."""
    import oracle
    N, C, H, W, k, d, s, combine, dtype = WORKLOADS[name]
    n_sub = min(N, 8)
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
        if el > budget_s or reps >= 200:
            break
    per = el / reps
    ab = algorithmic_bytes(n_sub, C, H, W, k, s, 4)
    return {
        'value': (ab['fwd'] + ab['bwd']) / per / 1e9, 'unit': 'GB/s', 'cores': threads,
        'kind': 'port',
        'sample': '%d of %d samples of %s in fp32, forward+backward, %d repetitions, '
                  '%.2f s each, C oracle with OpenMP' % (n_sub, N, name, reps, per),
        'images_per_s': n_sub / per,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=200)
    ap.add_argument('--warmup', type=int, default=20)
    ap.add_argument('--workload', default=DEFAULT_WORKLOAD, choices=sorted(WORKLOADS))
    ap.add_argument('--all', action='store_true', help='also time the other workloads (stderr)')
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg')
    args = ap.parse_args()
    if args.gpus != 1:
        log('bench.py measures one GPU: the operator shards over the batch with no exchange, '
            'and this build runs on a single device.  Re-run with --gpus 1.')
        sys.exit(2)
    assert torch.cuda.is_available(), 'bench.py needs a GPU'
    torch.cuda.set_device(0)
    from ddfnet_amd import _lib as lib
    lib.lib()

    extra = {}
    if args.all:
        for name in WORKLOADS:
            if name != args.workload:
                extra[name] = run_workload(name, args.steps, args.warmup, lib)
    res = run_workload(args.workload, args.steps, args.warmup, lib)

    dominant = max(res['phase_ms'], key=lambda p: res['phase_ms'][p]['mean'])
    dom_bytes = res['bytes'][dominant]
    dom_s = res['phase_ms'][dominant]['mean'] * 1e-3
    achieved = dom_bytes / dom_s / 1e9
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
        'pct_of_hbm_peak': round(100 * res['gbps'] / HBM_PEAK_GBPS, 2),
        'images_per_s': round(res['images_per_s'], 1),
        'roofline': {'bound': 'hbm', 'kernel': dominant, 'achieved': round(achieved, 2),
                     'peak': HBM_PEAK_GBPS, 'unit': 'GB/s',
                     'frac': round(achieved / HBM_PEAK_GBPS, 4), 'traffic': None,
                     'bytes_per_launch': dom_bytes,
                     'avg_launch_us': round(dom_s * 1e6, 3)},
        'phases_us': {p: round(v['mean'] * 1e3, 3) for p, v in res['phase_ms'].items()},
    }
    if extra:
        line['other_workloads'] = {
            n: {'gbps': round(r['gbps'], 1), 'us_per_step': round(r['ms_per_step'] * 1e3, 2),
                'images_per_s': round(r['images_per_s'], 1)} for n, r in extra.items()}
    if not args.no_cpu:
        line['cpu_baseline'] = cpu_baseline(args.workload)
        cb = line['cpu_baseline']
        cb['value'] = round(cb['value'], 3)
        cb['images_per_s'] = round(cb['images_per_s'], 1)
        log('[cpu] %s: %.2f GB/s on %d threads' % (cb['sample'], cb['value'], cb['cores']))
    print(json.dumps(line), flush=True)


if __name__ == '__main__':
    main()
