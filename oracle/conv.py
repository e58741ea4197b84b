"""TEST INFRASTRUCTURE: ctypes front end of the convolution oracle
(oracle/conv_oracle.c) and of the compiled reference im2col / col2im
(oracle/_ref/libref_conv.so, when built).

Reference followed: opzoo/Convolution/Convolution.cpp:13-120,
opzoo/Convolution/Convolution.py:17-84.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ORACLE_SO = os.path.join(_HERE, 'liboracle_conv.so')
_REF_SO = os.path.join(_HERE, '_ref', 'libref_conv.so')
_libs = {}


def _lib():
    if 'oracle' not in _libs:
        if not os.path.exists(_ORACLE_SO):
            subprocess.check_call(['make', '-C', _HERE, 'oracle'], stdout=subprocess.DEVNULL)
        _libs['oracle'] = ctypes.CDLL(_ORACLE_SO)
    return _libs['oracle']


def ref_available():
    return os.path.exists(_REF_SO)


def _ref():
    if 'ref' not in _libs:
        _libs['ref'] = ctypes.CDLL(_REF_SO)
    return _libs['ref']


def out_size(size, k, pad, stride, dil):
    """Convolution.py:69-72."""
    return (size + 2 * pad - ((k - 1) * dil + 1)) // stride + 1


def _ci(*vals):
    return [ctypes.c_int(int(v)) for v in vals]


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def im2col(im, kernel, pad, stride, dil, impl='oracle'):
    """im [C,H,W] -> col [C*KH*KW, OH, OW]."""
    im = np.ascontiguousarray(im, dtype=np.float32)
    C, H, W = im.shape
    OH, OW = out_size(H, kernel[0], pad[0], stride[0], dil[0]), out_size(W, kernel[1], pad[1], stride[1], dil[1])
    col = np.empty((C * kernel[0] * kernel[1], OH, OW), np.float32)
    geo = _ci(H, W, kernel[0], kernel[1], pad[0], pad[1], stride[0], stride[1], dil[0], dil[1], OH, OW)
    if impl == 'oracle':
        _lib().oracle_im2col_f32(ctypes.c_int(col.size), _p(im), *geo, _p(col))
    else:
        _ref().im2col_341af5d3(ctypes.c_int(-1), ctypes.c_int(col.size), _p(im), *geo, _p(col))
    return col


def col2im(col, im_shape, kernel, pad, stride, dil, impl='oracle'):
    """col [C*KH*KW, OH, OW] -> im [C,H,W]."""
    col = np.ascontiguousarray(col, dtype=np.float32)
    C, H, W = im_shape
    OH, OW = col.shape[1], col.shape[2]
    im = np.empty((C, H, W), np.float32)
    geo = _ci(H, W, kernel[0], kernel[1], pad[0], pad[1], stride[0], stride[1], dil[0], dil[1], OH, OW)
    if impl == 'oracle':
        _lib().oracle_col2im_f32(ctypes.c_int(im.size), _p(col), *geo, _p(im))
    else:
        _ref().col2im_341af5d3(ctypes.c_int(-1), ctypes.c_int(im.size), _p(col), *geo, _p(im))
    return im


def conv2d_forward(x, w, bias, pad, stride, dil):
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    N, C, H, W = x.shape
    D, _, KH, KW = w.shape
    OH, OW = out_size(H, KH, pad[0], stride[0], dil[0]), out_size(W, KW, pad[1], stride[1], dil[1])
    y = np.empty((N, D, OH, OW), np.float32)
    col = np.empty(C * KH * KW * OH * OW, np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    _lib().oracle_conv2d_forward_f32(_p(x), _p(w), _p(b) if b is not None else None,
                                     *_ci(N, C, H, W, D, KH, KW, pad[0], pad[1], stride[0], stride[1],
                                          dil[0], dil[1], OH, OW), _p(col), _p(y))
    return y


def conv2d_backward(dy, x, w, pad, stride, dil, with_bias=True):
    """-> dx, dw, db (db None unless with_bias)."""
    dy = np.ascontiguousarray(dy, dtype=np.float32)
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    N, C, H, W = x.shape
    D, _, KH, KW = w.shape
    OH, OW = dy.shape[2], dy.shape[3]
    dx, dw = np.empty_like(x), np.empty_like(w)
    db = np.empty(D, np.float32) if with_bias else None
    scratch = np.empty(2 * C * KH * KW * OH * OW, np.float32)
    _lib().oracle_conv2d_backward_f32(_p(dy), _p(x), _p(w),
                                      *_ci(N, C, H, W, D, KH, KW, pad[0], pad[1], stride[0], stride[1],
                                           dil[0], dil[1], OH, OW), _p(scratch), _p(dx), _p(dw),
                                      _p(db) if db is not None else None)
    return dx, dw, db
