"""Writes the golden ROIAlign vectors in this directory.

Expected outputs come from the COMPILED REFERENCE kernels (oracle/_ref, built by
oracle/Makefile from the reference checkout): forward from the OpenMP build,
backward from the single-thread build (fixed summation order).  Run it in a
container that has the reference checkout; the .npz files are what is committed.
    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import roialign as oracle  # noqa: E402


def case(name, seed, N, C, H, W, R, pooled, scale, S, span, adversarial=False):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    c = rng.uniform(0, span, size=(R, 2))
    wh = rng.uniform(1, span / 2, size=(R, 2))
    b = rng.integers(0, N, size=(R, 1))
    rois = np.concatenate([b, c - wh / 2, c + wh / 2], axis=1).astype(np.float32)
    if adversarial:
        rois[0, 1:] = [span * 3, span * 3, span * 4, span * 4]     # outside
        rois[1, 1:] = [span / 3, span / 3, span / 3, span / 3]     # zero size
        rois[2, 1:] = [7.3, 9.1, 7.6, 9.2]                         # sub-pixel
        rois[3, 1:] = [-span / 2, -span / 2, span / 2, span / 3]   # partly outside
        rois[4, 1:] = [span / 2, span / 2, span / 4, span / 4]     # reversed
        rois[5, 1:] = [0, 0, W / scale, H / scale]                 # whole map: samples at y == H edge
    dy = rng.standard_normal((R, C) + pooled).astype(np.float32)
    y = oracle.forward(x, rois, pooled, scale, S, impl='ref_omp')
    dx = oracle.backward(dy, rois, x.shape, scale, S, impl='ref_serial')
    np.savez_compressed(os.path.join(HERE, name + '.npz'), data=x, rois=rois, dy=dy, y=y, dx=dx,
                        pooled_size=np.array(pooled), spatial_scale=np.float64(scale),
                        sampling_ratio=np.int64(S))
    print(name, y.shape, dx.shape)


def case_f64(name, seed, N, C, H, W, R, pooled, scale, S, span):
    """The double instantiation: forward only (the reference cannot build its
    backward in double), written to the f64/ subdirectory."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((N, C, H, W))
    c = rng.uniform(0, span, size=(R, 2))
    wh = rng.uniform(1, span / 2, size=(R, 2))
    b = rng.integers(0, N, size=(R, 1))
    rois = np.concatenate([b, c - wh / 2, c + wh / 2], axis=1)
    rois[0, 1:] = [span * 3, span * 3, span * 4, span * 4]     # outside
    rois[1, 1:] = [span / 3, span / 3, span / 3, span / 3]     # zero size
    rois[2, 1:] = [7.3, 9.1, 7.6, 9.2]                         # sub-pixel
    rois[3, 1:] = [-span / 2, -span / 2, span / 2, span / 3]   # partly outside
    rois[4, 1:] = [0, 0, W / scale, H / scale]                 # whole map
    y = oracle.forward_f64(x, rois, pooled, scale, S, impl='ref_omp')
    os.makedirs(os.path.join(HERE, 'f64'), exist_ok=True)
    np.savez_compressed(os.path.join(HERE, 'f64', name + '.npz'), data=x, rois=rois, y=y,
                        pooled_size=np.array(pooled), spatial_scale=np.float64(scale),
                        sampling_ratio=np.int64(S))
    print(name, y.shape)


if __name__ == '__main__':
    assert oracle.ref_available('serial'), 'build oracle/_ref first (make -C oracle ref)'
    case('roialign_s2_7x7', 1, N=2, C=6, H=24, W=40, R=24, pooled=(7, 7), scale=0.25, S=2, span=150.0)
    case('roialign_s0_3x4', 2, N=5, C=3, H=16, W=16, R=16, pooled=(3, 4), scale=16 / 224, S=0, span=224.0)
    case('roialign_adversarial_14x14', 3, N=3, C=4, H=20, W=20, R=20, pooled=(14, 14), scale=0.125,
         S=2, span=160.0, adversarial=True)
    case('roialign_s3_2x5', 4, N=1, C=2, H=9, W=31, R=10, pooled=(2, 5), scale=0.5, S=3, span=60.0,
         adversarial=True)
    case_f64('roialign_f64_s2_7x7', 11, N=2, C=3, H=18, W=25, R=12, pooled=(7, 7), scale=0.25, S=2, span=100.0)
    case_f64('roialign_f64_s0_3x4', 12, N=2, C=2, H=16, W=16, R=10, pooled=(3, 4), scale=16 / 224, S=0, span=224.0)
