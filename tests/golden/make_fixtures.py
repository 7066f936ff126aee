"""Writes the known-answer fixtures of this folder.

The reference ships no golden vectors and cannot run here (CUDA-only, no CPU
path), so these vectors come from this build's own CPU oracle - the literal
loop form of the operator and torch autograd through the unfold form, both in
fp64, which tests/test_oracle.py pins with closed forms and invariants.  They
are regression data: they freeze today's oracle so that a later change to it
(or to the kernels) that alters any result shows up as a fixture mismatch.

Each file holds inputs and expected results of one small case:
    x, cf, sf, go            inputs (fp64, drawn from N(0,1), seeded)
    out, dx, dcf, dsf        forward result and the three gradients (fp64)
    k, d, s, combine         kernel size, dilation, stride, 0 = mul / 1 = add

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), '..', '..'))
import oracle  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

# name: (N, C, H, W, k, d, s, combine)
CASES = {
    'mul_k3': (1, 4, 7, 9, 3, 1, 1, 'mul'),
    'add_k3': (1, 4, 7, 9, 3, 1, 1, 'add'),
    'mul_k3_d2': (1, 3, 8, 8, 3, 2, 1, 'mul'),
    'mul_k3_s2_odd': (2, 3, 9, 7, 3, 1, 2, 'mul'),
    'add_k5_d2': (1, 2, 10, 10, 5, 2, 1, 'add'),
    'mul_k5_s2': (1, 2, 9, 10, 5, 1, 2, 'mul'),
    'mul_k1': (2, 3, 5, 6, 1, 1, 1, 'mul'),
    'mul_k7': (1, 2, 7, 7, 7, 1, 1, 'mul'),
}


def main():
    for seed, (name, (N, C, H, W, k, d, s, combine)) in enumerate(sorted(CASES.items())):
        x, cf, sf, go = oracle.make_inputs(N, C, H, W, k, s, torch.float64, standardize=False,
                                           seed=100 + seed)
        out = oracle.loop_forward(x, cf, sf, k, d, s, combine)
        dx, dcf, dsf = oracle.unfold_backward(go, x, cf, sf, k, d, s, combine)
        np.savez_compressed(
            os.path.join(HERE, name + '.npz'),
            x=x.numpy(), cf=cf.numpy(), sf=sf.numpy(), go=go.numpy(), out=out.numpy(),
            dx=dx.numpy(), dcf=dcf.numpy(), dsf=dsf.numpy(),
            k=k, d=d, s=s, combine=0 if combine == 'mul' else 1)
        print(name, tuple(out.shape))


if __name__ == '__main__':
    main()
