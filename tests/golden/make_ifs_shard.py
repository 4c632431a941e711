#!/usr/bin/env python3
"""Writes tests/golden/ifs_cfg5_shard.npz: the input of BASELINE.json's config 5 at full size -- one 128-cube sample of
three random 3-D iterated function systems (4 affine maps each, contraction 0.3 .. 0.7, 2e5 iterations per fractal,
seed 5000), voxelised by ``oracle.ifs_volume``, of which one rank's depth shard (the first 64 planes) is kept as class
labels (uint8, 0 = background; the occupancy volume the network reads is ``labels > 0``).

bench.py and the full-size tests read this file, so that the GPU step and the host stock arm see the same bits without
the product path importing the oracle; ``tests/test_oracle.py`` checks the file against the generator.
Run from the repository root:  python tests/golden/make_ifs_shard.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as orc  # noqa: E402

GRID, DEPTH, ITERATIONS, SEED = 128, 64, 200_000, 5000


def shard_labels():
    _occ, lab = orc.ifs_volume(GRID, iterations=ITERATIONS, seed=SEED)
    return lab[0, :DEPTH].numpy().astype(np.uint8)


def main():
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ifs_cfg5_shard.npz")
    labels = shard_labels()
    np.savez_compressed(path, labels=labels, grid=GRID, depth=DEPTH, iterations=ITERATIONS, seed=SEED)
    print(f"wrote {path}: {labels.shape}, {float((labels > 0).mean()):.4f} occupied, classes {sorted(set(labels.ravel().tolist()))}")


if __name__ == "__main__":
    main()
