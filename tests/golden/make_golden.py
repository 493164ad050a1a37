"""Writes the committed fixtures in this folder.  Run from the repository root:
    python tests/golden/make_golden.py
Inputs are seeded; expected outputs come from exact rational arithmetic (hash) or float64 brute
force (attention), not from the code under test.  The reference has no fixtures of its own for
this path (its tests only print), so these are the golden vectors."""
import os
import sys
from fractions import Fraction

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))


def exact_buckets(x, proj):
    """Gray-coded sign pattern from exact rational dot products."""
    n, d = x.shape
    r = proj.shape[1]
    out = np.zeros(n, dtype=np.int32)
    xs = [[Fraction(float(v)) for v in row] for row in x]
    ps = [[Fraction(float(proj[k, j])) for k in range(d)] for j in range(r)]
    for i in range(n):
        b = 0
        for j in range(r):
            if sum(a * c for a, c in zip(xs[i], ps[j])) > 0:
                b |= 1 << j
        out[i] = b ^ (b >> 1)
    return out


def main():
    g = torch.Generator().manual_seed(20240607)
    x = torch.randn((1, 2, 192, 64), generator=g).half()
    # rows that stress the sign decision: zeros, exact cancellation, tiny values, huge values
    x[0, 0, 0] = 0
    x[0, 0, 1, :32] = x[0, 0, 1, 32:]
    x[0, 0, 2] *= 2.0 ** -14
    x[0, 1, 3] *= 2.0 ** 9
    proj = torch.randn((64, 8), generator=g).half()
    proj[32:, 0] = -proj[:32, 0]  # makes row (0,0,1) cancel exactly on projection 0
    buckets = np.stack([exact_buckets(x[0, h].double().numpy(), proj.double().numpy()) for h in range(2)])[None]
    np.savez_compressed(os.path.join(HERE, "lsh_hash_fp16.npz"), x=x.view(torch.int16).numpy(),
                        proj=proj.view(torch.int16).numpy(), buckets=buckets)
    print("wrote lsh_hash_fp16.npz", buckets.shape, int(buckets[0, 0, 0]), int(buckets[0, 0, 1]))


if __name__ == "__main__":
    main()
