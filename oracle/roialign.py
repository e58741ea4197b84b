"""TEST INFRASTRUCTURE: ctypes front end of the CPU oracle (oracle/roialign_oracle.c)
and of the compiled reference kernels (oracle/_ref, when built), plus a slow,
independent NumPy loop used to pin the C restatement on tiny shapes.

Reference followed: opzoo/ROIAlign/ROIAlign.cpp:9-161, opzoo/ROIAlign/bilinear.h:10-112.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ORACLE_SO = os.path.join(_HERE, 'liboracle_roialign.so')
_REF_SO = {
    'omp': os.path.join(_HERE, '_ref', 'libref_roialign_omp.so'),
    'serial': os.path.join(_HERE, '_ref', 'libref_roialign_serial.so'),
}
_libs = {}


def build(with_ref=True):
    """Compile the oracle (and oracle/_ref if the reference checkout exists)."""
    target = 'all' if with_ref else 'oracle'
    subprocess.check_call(['make', '-C', _HERE, target], stdout=subprocess.DEVNULL)


def _lib():
    if 'oracle' not in _libs:
        if not os.path.exists(_ORACLE_SO):
            build(with_ref=False)
        _libs['oracle'] = ctypes.CDLL(_ORACLE_SO)
    return _libs['oracle']


def ref_available(kind='omp'):
    return os.path.exists(_REF_SO[kind])


def _ref(kind):
    key = 'ref_' + kind
    if key not in _libs:
        _libs[key] = ctypes.CDLL(_REF_SO[kind])
    return _libs[key]


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(ctypes.c_void_p)


def _common_args(n_out, ptr_a, scale, C, H, W, PH, PW, S):
    return [ctypes.c_int(n_out), ptr_a, ctypes.c_float(scale), ctypes.c_int(C),
            ctypes.c_int(H), ctypes.c_int(W), ctypes.c_int(PH), ctypes.c_int(PW),
            ctypes.c_int(S)]


def num_threads():
    return int(_lib().oracle_num_threads())


def forward(data, rois, pooled_size, spatial_scale, sampling_ratio, impl='oracle'):
    """y[R,C,PH,PW] for NCHW fp32 `data` and rois[R,5]; impl: oracle | ref_omp | ref_serial."""
    data, pd = _f32(data)
    rois, pr = _f32(rois)
    _, C, H, W = data.shape
    PH, PW = pooled_size
    out = np.empty((rois.shape[0], C, PH, PW), dtype=np.float32)
    args = _common_args(out.size, pd, spatial_scale, C, H, W, PH, PW, sampling_ratio)
    args += [pr, out.ctypes.data_as(ctypes.c_void_p)]
    if impl == 'oracle':
        _lib().oracle_roi_align_forward_f32(*args)
    else:
        _ref(impl[4:]).roi_align_forward_ab78de3c(ctypes.c_int(-1), *args)
    return out


def _f64(a):
    a = np.ascontiguousarray(a, dtype=np.float64)
    return a, a.ctypes.data_as(ctypes.c_void_p)


def forward_f64(data, rois, pooled_size, spatial_scale, sampling_ratio, impl='oracle'):
    """The double instantiation: float64 `data`, `rois` and scale.  impl: oracle |
    ref_omp | ref_serial (the compiled reference, forward only)."""
    data, pd = _f64(data)
    rois, pr = _f64(rois)
    N, C, H, W = data.shape
    PH, PW = pooled_size
    R = rois.shape[0]
    out = np.zeros((R, C, PH, PW), dtype=np.float64)
    po = out.ctypes.data_as(ctypes.c_void_p)
    geometry = [ctypes.c_double(spatial_scale)] + [ctypes.c_int(v) for v in (C, H, W, PH, PW, sampling_ratio)]
    if impl == 'oracle':
        _lib().oracle_roi_align_forward_f64(ctypes.c_int(R), ctypes.c_int(N), pd, *geometry, pr, po)
    else:
        _ref(impl[4:]).roi_align_forward_6b9e6c9b(ctypes.c_int(-1), ctypes.c_int(out.size), pd, *geometry,
                                                  pr, po)
    return out


def backward_f64(dy, rois, data_shape, spatial_scale, sampling_ratio, dx=None):
    """dx[N,C,H,W] in float64, accumulated into `dx` (zeros if None); oracle only."""
    dy, pdy = _f64(dy)
    rois, pr = _f64(rois)
    N, C, H, W = data_shape
    PH, PW = dy.shape[2], dy.shape[3]
    if dx is None:
        dx = np.zeros(data_shape, dtype=np.float64)
    assert dx.dtype == np.float64 and dx.flags.c_contiguous
    geometry = [ctypes.c_double(spatial_scale)] + [ctypes.c_int(v) for v in (C, H, W, PH, PW, sampling_ratio)]
    _lib().oracle_roi_align_backward_f64(ctypes.c_int(rois.shape[0]), ctypes.c_int(N), pdy, *geometry,
                                         dx.ctypes.data_as(ctypes.c_void_p), pr)
    return dx


def backward(dy, rois, data_shape, spatial_scale, sampling_ratio, impl='oracle', dx=None):
    """dx[N,C,H,W] accumulated into `dx` (zeros if None).

    impl: oracle (reference schedule, omp atomic) | ordered (fixed summation
    order) | ref_omp | ref_serial."""
    dy, pdy = _f32(dy)
    rois, pr = _f32(rois)
    N, C, H, W = data_shape
    PH, PW = dy.shape[2], dy.shape[3]
    if dx is None:
        dx = np.zeros(data_shape, dtype=np.float32)
    assert dx.dtype == np.float32 and dx.flags.c_contiguous
    pdx = dx.ctypes.data_as(ctypes.c_void_p)
    args = _common_args(dy.size, pdy, spatial_scale, C, H, W, PH, PW, sampling_ratio)
    args += [pdx, pr]
    if impl == 'oracle':
        _lib().oracle_roi_align_backward_f32(*args)
    elif impl == 'ordered':
        _lib().oracle_roi_align_backward_f32_ordered(*args, ctypes.c_int(N))
    else:
        _ref(impl[4:]).roi_align_backward_f318a24e(ctypes.c_int(-1), *args)
    return dx


# ---------------------------------------------------------------------------
# Independent slow restatement (NumPy scalars of one type, explicit loops).  Written
# from the algorithm description, structured differently from the C file (it
# builds per-axis sample tables first), so a slip in either shows up as a
# mismatch.  Tiny shapes only.
# ---------------------------------------------------------------------------
def _axis_table(start, bin_size, pooled, grid, size, _F):
    """Per (p, i): (valid, low, high, l, h) along one axis."""
    table = []
    for p in range(pooled):
        for i in range(grid):
            v = _F(_F(start + _F(_F(p) * bin_size)) +
                   _F(_F(_F(_F(i) + _F(0.5)) * bin_size) / _F(grid)))
            if v < _F(-1.0) or v > _F(size):
                table.append((False, 0, 0, _F(0), _F(0)))
                continue
            if v <= 0:
                v = _F(0)
            low = int(v)
            if low >= size - 1:
                low = high = size - 1
                v = _F(low)
            else:
                high = low + 1
            l = _F(v - _F(low))
            table.append((True, low, high, l, _F(_F(1) - l)))
    return table


def brute_force(data, rois, pooled_size, spatial_scale, sampling_ratio, dy=None, dtype=np.float32):
    """Returns (y, dx); dx is None when dy is None.  Every operation is rounded to
    `dtype` (float32: the reference's float kernels, float64: its double ones)."""
    _F = dtype
    data = np.asarray(data, dtype=_F)
    rois = np.asarray(rois, dtype=_F)
    N, C, H, W = data.shape
    PH, PW = pooled_size
    R = rois.shape[0]
    y = np.zeros((R, C, PH, PW), dtype=_F)
    dx = None if dy is None else np.zeros_like(data)
    scale = _F(spatial_scale)
    for r in range(R):
        b = int(rois[r, 0])
        sw, sh, ew, eh = (_F(rois[r, k] * scale) for k in (1, 2, 3, 4))
        rw = max(_F(ew - sw), _F(1))
        rh = max(_F(eh - sh), _F(1))
        bh, bw = _F(rh / _F(PH)), _F(rw / _F(PW))
        gh = sampling_ratio if sampling_ratio > 0 else int(np.ceil(_F(rh / _F(PH))))
        gw = sampling_ratio if sampling_ratio > 0 else int(np.ceil(_F(rw / _F(PW))))
        cnt = _F(gh * gw)
        ty = _axis_table(sh, bh, PH, gh, H, _F)
        tx = _axis_table(sw, bw, PW, gw, W, _F)
        for c in range(C):
            plane = data[b, c]
            for ph in range(PH):
                for pw in range(PW):
                    acc = _F(0)
                    for iy in range(gh):
                        vy, yl, yh, ly, hy = ty[ph * gh + iy]
                        for ix in range(gw):
                            vx, xl, xh, lx, hx = tx[pw * gw + ix]
                            if not (vy and vx):
                                continue
                            w = (_F(hy * hx), _F(hy * lx), _F(ly * hx), _F(ly * lx))
                            pos = ((yl, xl), (yl, xh), (yh, xl), (yh, xh))
                            val = _F(0)
                            for k in range(4):
                                val = _F(val + _F(w[k] * plane[pos[k]]))
                            acc = _F(acc + val)
                            if dy is not None:
                                g = dy[r, c, ph, pw]
                                for k in range(4):
                                    dx[b, c][pos[k]] = _F(dx[b, c][pos[k]] +
                                                          _F(_F(g * w[k]) / cnt))
                    y[r, c, ph, pw] = _F(acc / cnt)
    return y, dx
