#!/usr/bin/env python3
"""Writes tests/golden/hotpath_small.npz: small seeded problems of every op on the hot path together
with the answers of the plain-C brute-force loops in oracle/conv_ref.c (not torch), so that the torch
oracle, the C oracle and the HIP kernels can each be checked against a fixed, committed answer.

The reference repository holds no numeric vectors for this path (its fixtures are shape corpora and
timings), so these are generated here; run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import cref  # noqa: E402


def ints(shape, seed, lo=-2, hi=3):
    return torch.randint(lo, hi, shape, generator=torch.Generator().manual_seed(seed)).double()


def main():
    out = {}
    # conv3d 3x3x3, padding (0,1,1) (the depth-shard form), with bias
    x = ints((2, 4, 5, 6, 7), 1)
    w = ints((3, 4, 3, 3, 3), 2)
    b = ints((3,), 3)
    gy = ints((2, 3, 3, 6, 7), 4)
    out.update(conv_x=x, conv_w=w, conv_b=b, conv_gy=gy,
               conv_y=cref.conv3d_fwd(x, w, b, (1, 1, 1), (0, 1, 1)),
               conv_gx=cref.conv3d_dgrad(gy, w, x.shape, (1, 1, 1), (0, 1, 1)),
               conv_gw=cref.conv3d_wgrad(x, w.shape, gy, (1, 1, 1), (0, 1, 1)))
    # strided, dilated, anisotropic
    x2 = ints((1, 3, 7, 8, 9), 5)
    w2 = ints((2, 3, 2, 3, 1), 6)
    out.update(sconv_x=x2, sconv_w=w2, sconv_y=cref.conv3d_fwd(x2, w2, None, (2, 1, 3), (1, 0, 2), (1, 2, 1)))
    gy2 = ints(tuple(out["sconv_y"].shape), 7)
    out.update(sconv_gy=gy2, sconv_gw=cref.conv3d_wgrad(x2, w2.shape, gy2, (2, 1, 3), (1, 0, 2), (1, 2, 1)))
    # transposed conv k == s == 2
    xt = ints((1, 3, 2, 3, 2), 8)
    wt = ints((3, 4, 2, 2, 2), 9)
    bt = ints((4,), 10)
    out.update(convt_x=xt, convt_w=wt, convt_b=bt, convt_y=cref.convT3d_fwd(xt, wt, bt))
    # GroupNorm + ReLU forward / backward
    g = torch.Generator().manual_seed(11)
    xg = torch.randn((2, 8, 3, 4, 5), generator=g, dtype=torch.float64) * 2 + 0.7
    gamma = 1 + 0.3 * torch.randn(8, generator=g, dtype=torch.float64)
    beta = 0.2 * torch.randn(8, generator=g, dtype=torch.float64)
    dy = torch.randn((2, 8, 3, 4, 5), generator=g, dtype=torch.float64)
    y, mean, rstd = cref.groupnorm_fwd(xg, 4, gamma, beta, 1e-5, True)
    dx, dgamma, dbeta = cref.groupnorm_bwd(dy, xg, 4, gamma, beta, mean, rstd, True)
    out.update(gn_x=xg, gn_gamma=gamma, gn_beta=beta, gn_dy=dy, gn_y=y, gn_mean=mean, gn_rstd=rstd, gn_dx=dx,
               gn_dgamma=dgamma, gn_dbeta=dbeta)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hotpath_small.npz")
    np.savez_compressed(path, **{k: np.ascontiguousarray(v.numpy()) for k, v in out.items()})
    print("wrote", path, {k: tuple(v.shape) for k, v in out.items()})


if __name__ == "__main__":
    main()
