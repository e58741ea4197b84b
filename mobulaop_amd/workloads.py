"""Seeded synthetic ROIAlign workloads (the benchmark / parity configurations).

Each generator returns a dict with NumPy arrays `data` (NCHW), `rois`
([R,5] rows `[batch_idx, x1, y1, x2, y2]` in image pixels, always fp32), `dy`
(N(0,1), shape [R,C,PH,PW]) and the operator parameters `pooled_size`,
`spatial_scale`, `sampling_ratio`.  `scale_down` shrinks channel and ROI counts
(not the geometry) so the CPU checker finishes quickly in tests.
"""
import numpy as np

__all__ = ['WORKLOADS', 'make_workload', 'algorithmic_bytes', 'touched_fraction', 'gather_bytes']


def _pack(data, rois, pooled, scale, ratio, rng, name, dy=True):
    R, C = rois.shape[0], data.shape[1]
    out = dict(name=name, data=data, rois=rois.astype(np.float32), pooled_size=pooled,
               spatial_scale=scale, sampling_ratio=ratio)
    out['dy'] = rng.standard_normal((R, C, pooled[0], pooled[1]), dtype=np.float32) if dy else None
    return out


def _uniform_boxes(rng, R, extent, nbatch):
    p = rng.uniform(0, extent, size=(R, 2, 2)).astype(np.float32)  # [R, point, (x,y)]
    for _ in range(8):  # resample ties so that x1<x2 and y1<y2
        tie = (p[:, 0, 0] == p[:, 1, 0]) | (p[:, 0, 1] == p[:, 1, 1])
        if not tie.any():
            break
        p[tie] = rng.uniform(0, extent, size=(int(tie.sum()), 2, 2)).astype(np.float32)
    lo, hi = p.min(axis=1), p.max(axis=1)
    b = rng.integers(0, nbatch, size=R).astype(np.float32)
    return np.stack([b, lo[:, 0], lo[:, 1], hi[:, 0], hi[:, 1]], axis=1)


def cfg1(C=256, R=512, seed=1001):
    """2xCx64x64 U[0,1); uniform boxes in [0,512)^2; scale 1/8; 7x7; S=2."""
    rng = np.random.default_rng(seed)
    data = rng.random((2, C, 64, 64), dtype=np.float32)
    rois = _uniform_boxes(rng, R, 512.0, 2)
    return _pack(data, rois, (7, 7), 1.0 / 8, 2, rng, 'cfg1')


def cfg2(C=256, R=4000, seed=1002):
    """FPN-P2 like: 4xCx200x336 U[0,1); log-uniform 16..512 px boxes inside a
    1344x800 (WxH) image; scale 1/4; 7x7; S=2."""
    rng = np.random.default_rng(seed)
    data = rng.random((4, C, 200, 336), dtype=np.float32)
    w = np.exp(rng.uniform(np.log(16.0), np.log(512.0), size=R))
    h = np.exp(rng.uniform(np.log(16.0), np.log(512.0), size=R))
    cx = rng.uniform(w / 2, 1344.0 - w / 2)
    cy = rng.uniform(h / 2, 800.0 - h / 2)
    b = rng.integers(0, 4, size=R)
    rois = np.stack([b, cx - w / 2, cy - h / 2, cx + w / 2, cy + h / 2], axis=1)
    return _pack(data, rois, (7, 7), 1.0 / 4, 2, rng, 'cfg2')


def cfg3(C=256, R=8192, seed=1003):
    """Mask-head: 8xCx128x128 (1024^2 image); ROI centres from 16 Gaussian
    clusters per image (sigma 32 px), sizes log-uniform 32..512; a random 10 %
    are adversarial (partly outside, zero-width/height, sub-pixel); scale 1/8;
    14x14; S=2."""
    rng = np.random.default_rng(seed)
    N = 8
    data = rng.random((N, C, 128, 128), dtype=np.float32)
    centres = rng.uniform(0, 1024.0, size=(N, 16, 2))
    b = rng.integers(0, N, size=R)
    k = rng.integers(0, 16, size=R)
    c = centres[b, k] + rng.normal(0, 32.0, size=(R, 2))
    w = np.exp(rng.uniform(np.log(32.0), np.log(512.0), size=R))
    h = np.exp(rng.uniform(np.log(32.0), np.log(512.0), size=R))
    x1, y1, x2, y2 = c[:, 0] - w / 2, c[:, 1] - h / 2, c[:, 0] + w / 2, c[:, 1] + h / 2
    adv = rng.permutation(R)[:R // 10]
    third = np.array_split(adv, 3)
    # (a) shifted partially outside the map
    sx = rng.choice([-1.0, 1.0], size=third[0].size) * rng.uniform(600, 1100, size=third[0].size)
    sy = rng.choice([-1.0, 1.0], size=third[0].size) * rng.uniform(600, 1100, size=third[0].size)
    x1[third[0]] += sx
    x2[third[0]] += sx
    y1[third[0]] += sy
    y2[third[0]] += sy
    # (b) zero width or height
    zw = third[1][::2]
    zh = third[1][1::2]
    x2[zw] = x1[zw]
    y2[zh] = y1[zh]
    # (c) sub-pixel boxes
    x2[third[2]] = x1[third[2]] + rng.uniform(0.01, 0.99, size=third[2].size)
    y2[third[2]] = y1[third[2]] + rng.uniform(0.01, 0.99, size=third[2].size)
    rois = np.stack([b, x1, y1, x2, y2], axis=1)
    return _pack(data, rois, (14, 14), 1.0 / 8, 2, rng, 'cfg3')


def cfg4(C=512, R=6000, seed=1004):
    """Inference: 4xCx100x100 N(0,1) stored as fp16 (1600^2 image); uniform
    boxes; rois fp32; scale 1/16; 7x7; adaptive sampling (S=0); forward only."""
    rng = np.random.default_rng(seed)
    data = rng.standard_normal((4, C, 100, 100), dtype=np.float32).astype(np.float16)
    rois = _uniform_boxes(rng, R, 1600.0, 4)
    return _pack(data, rois, (7, 7), 1.0 / 16, 0, rng, 'cfg4', dy=False)


WORKLOADS = dict(cfg1=cfg1, cfg2=cfg2, cfg3=cfg3, cfg4=cfg4)


def make_workload(name, scale_down=1):
    """Build a workload; `scale_down` divides both C and R (geometry untouched)."""
    fn = WORKLOADS[name]
    if scale_down == 1:
        return fn()
    import inspect
    d = {k: v.default for k, v in inspect.signature(fn).parameters.items()}
    return fn(C=max(1, d['C'] // scale_down), R=max(1, d['R'] // scale_down))


def algorithmic_bytes(w):
    """Compulsory HBM bytes (each tensor once): returns (fwd, bwd).

    fwd = e*|x| + 20*R + e*|y| ;  bwd = e*|dy| + 20*R + e*|dx|  (the dx term is
    one full write and covers the zero-initialisation)."""
    e = w['data'].dtype.itemsize
    nx = w['data'].size
    R, C = w['rois'].shape[0], w['data'].shape[1]
    ny = R * C * w['pooled_size'][0] * w['pooled_size'][1]
    b = e * nx + 20 * R + e * ny
    return b, b


def touched_fraction(w):
    """Fraction of the map's pixels (one pixel of a channel block = one 128-byte
    line of the blocked layout) inside the box of at least one ROI: what part of
    the e*|x| term of the algorithmic bytes the ROIs can actually reach."""
    N, _, H, W = w['data'].shape
    hit = np.zeros((N, H, W), dtype=bool)
    s = w['spatial_scale']
    for b, x1, y1, x2, y2 in w['rois']:
        b = int(b)
        if b < 0 or b >= N:
            continue
        xa, ya = x1 * s, y1 * s
        xb, yb = xa + max(x2 * s - xa, 1.0), ya + max(y2 * s - ya, 1.0)
        c0, c1 = int(np.floor(max(xa, 0.0))), int(np.floor(min(xb, W - 1))) + 1
        r0, r1 = int(np.floor(max(ya, 0.0))), int(np.floor(min(yb, H - 1))) + 1
        if c0 < W and r0 < H and c1 >= 0 and r1 >= 0:
            hit[b, max(r0, 0):min(r1 + 1, H), max(c0, 0):min(c1 + 1, W)] = True
    return float(hit.mean())


def gather_bytes(w):
    """Bytes a kernel without any reuse would pull through the caches in one
    forward pass: four corner values for each sample of each output,
    4 * e * S_h * S_w per output (the adaptive grid is ceil(roi/pooled) per ROI)."""
    e = w['data'].dtype.itemsize
    C = w['data'].shape[1]
    PH, PW = w['pooled_size']
    S = w['sampling_ratio']
    rois = w['rois'].astype(np.float32)
    if S > 0:
        samples = np.full(rois.shape[0], S * S, dtype=np.int64)
    else:
        s = np.float32(w['spatial_scale'])
        rw = np.maximum(rois[:, 3] * s - rois[:, 1] * s, np.float32(1))
        rh = np.maximum(rois[:, 4] * s - rois[:, 2] * s, np.float32(1))
        samples = (np.ceil(rh / np.float32(PH)) * np.ceil(rw / np.float32(PW))).astype(np.int64)
    return int(4 * e * C * PH * PW * samples.sum())
