"""Direct ctypes calls into the launcher library's C ABI with torch-owned device
memory: no Python binding in between.  Used by the GPU tests and by bench.py."""
import ctypes

import numpy as np
import torch

from mobulaop_amd import native

IMPL = {'auto': 0, 'tiled': 1, 'naive': 2}

# symbol suffixes of the storage types that take fp32 boxes: forward / forward_nhwc,
# backward, backward_assign
_SUFFIX = {torch.float32: ('ab78de3c', 'f318a24e', 'a8793cbe'),
           torch.float16: ('e874c59a', '23175303', '7924dbc8'),
           torch.bfloat16: ('f951d439', '0c43e974', '86156afd')}


def _ptr(t):
    assert t.is_contiguous()
    return ctypes.c_void_p(t.data_ptr())


def _begin(extents, stream=None):
    lib = native.library()
    if stream is None:
        lib.mobula_hip_set_stream(None, 1)
    else:
        lib.mobula_hip_set_stream(ctypes.c_void_p(stream), 0)
    if extents is not None:
        arr = (ctypes.c_longlong * len(extents))(*extents)
        lib.mobula_hip_set_arg_extents(arr, len(extents))
    return lib


def _end(lib):
    msg = lib.mobula_hip_last_error()
    if msg:
        lib.mobula_hip_clear_error()
        raise RuntimeError(msg.decode())


def _geom(scale, C, H, W, PH, PW, S, real=ctypes.c_float):
    return [real(scale)] + [ctypes.c_int(v) for v in (C, H, W, PH, PW, S)]


def forward(x, rois, pooled, scale, S, declare_extents=True, stream=None, dev=0):
    """x: torch cuda tensor [N,C,H,W] (fp32 or fp16), rois: cuda fp32 [R,5]."""
    N, C, H, W = x.shape
    PH, PW = pooled
    R = rois.shape[0]
    y = torch.empty((R, C, PH, PW), dtype=x.dtype, device=x.device)
    ext = [-1, x.numel(), -1, -1, -1, -1, -1, -1, -1, rois.numel(), y.numel()]
    lib = _begin(ext if declare_extents else [], stream)
    if x.dtype == torch.float64:   # the double instantiation: boxes and scale are double too
        assert rois.dtype == torch.float64
        lib.roi_align_forward_6b9e6c9b(ctypes.c_int(dev), ctypes.c_int(y.numel()), _ptr(x),
                                       *_geom(scale, C, H, W, PH, PW, S, ctypes.c_double), _ptr(rois), _ptr(y))
        _end(lib)
        return y
    fn = getattr(lib, 'roi_align_forward_' + _SUFFIX[x.dtype][0])
    fn(ctypes.c_int(dev), ctypes.c_int(y.numel()), _ptr(x), *_geom(scale, C, H, W, PH, PW, S),
       _ptr(rois), _ptr(y))
    _end(lib)
    return y


def forward_noalloc(x, rois, pooled, scale, S, y=None, stream=None, dev=0):
    """The entry point that allocates nothing; fp32 device tensors.  y may be given
    (a caller that cannot allocate brings its own output)."""
    N, C, H, W = x.shape
    PH, PW = pooled
    R = rois.shape[0]
    if y is None:
        y = torch.empty((R, C, PH, PW), dtype=x.dtype, device=x.device)
    ext = [-1, x.numel(), -1, -1, -1, -1, -1, -1, -1, -1, rois.numel(), y.numel()]
    lib = _begin(ext, stream)
    lib.roi_align_forward_noalloc_83212f20(ctypes.c_int(dev), ctypes.c_int(y.numel()), _ptr(x),
                                           *_geom(scale, C, H, W, PH, PW, S), ctypes.c_int(N),
                                           _ptr(rois), _ptr(y))
    _end(lib)
    return y


def backward(dy, rois, shape, scale, S, dx=None, assign=False, declare_extents=True, stream=None,
             dev=0):
    N, C, H, W = shape
    PH, PW = dy.shape[2], dy.shape[3]
    if dx is None:
        dx = (torch.full(shape, float('nan'), dtype=dy.dtype, device=dy.device) if assign
              else torch.zeros(shape, dtype=dy.dtype, device=dy.device))
    lib = native.library()
    if dy.dtype == torch.float64:
        assert rois.dtype == torch.float64
        geom = _geom(scale, C, H, W, PH, PW, S, ctypes.c_double)
        if assign:
            _begin([-1, dy.numel(), -1, -1, -1, -1, -1, -1, -1, -1, dx.numel(), rois.numel()]
                   if declare_extents else [], stream)
            lib.roi_align_backward_assign_4620f85e(ctypes.c_int(dev), ctypes.c_int(dy.numel()), _ptr(dy), *geom,
                                                   ctypes.c_int(N), _ptr(dx), _ptr(rois))
        else:
            _begin([-1, dy.numel(), -1, -1, -1, -1, -1, -1, -1, dx.numel(), rois.numel()]
                   if declare_extents else [], stream)
            lib.roi_align_backward_2b6c6dfa(ctypes.c_int(dev), ctypes.c_int(dy.numel()), _ptr(dy), *geom,
                                            _ptr(dx), _ptr(rois))
        _end(lib)
        return dx
    if assign:
        ext = [-1, dy.numel(), -1, -1, -1, -1, -1, -1, -1, -1, dx.numel(), rois.numel()]
        _begin(ext if declare_extents else [], stream)
        getattr(lib, 'roi_align_backward_assign_' + _SUFFIX[dy.dtype][2])(
            ctypes.c_int(dev), ctypes.c_int(dy.numel()), _ptr(dy), *_geom(scale, C, H, W, PH, PW, S),
            ctypes.c_int(N), _ptr(dx), _ptr(rois))
    else:
        ext = [-1, dy.numel(), -1, -1, -1, -1, -1, -1, -1, dx.numel(), rois.numel()]
        _begin(ext if declare_extents else [], stream)
        getattr(lib, 'roi_align_backward_' + _SUFFIX[dy.dtype][1])(
            ctypes.c_int(dev), ctypes.c_int(dy.numel()), _ptr(dy), *_geom(scale, C, H, W, PH, PW, S),
            _ptr(dx), _ptr(rois))
    _end(lib)
    return dx


def forward_nhwc(x, rois, pooled, scale, S, dev=0, stream=None):
    """x: cuda tensor [N,H,W,C] (fp32 or fp16); returns y [R,PH,PW,C]."""
    N, H, W, C = x.shape
    PH, PW = pooled
    R = rois.shape[0]
    y = torch.empty((R, PH, PW, C), dtype=x.dtype, device=x.device)
    ext = [-1, x.numel(), -1, -1, -1, -1, -1, -1, -1, rois.numel(), y.numel()]
    lib = _begin(ext, stream)
    fn = getattr(lib, 'roi_align_forward_nhwc_' + _SUFFIX[x.dtype][0])
    fn(ctypes.c_int(dev), ctypes.c_int(y.numel()), _ptr(x), *_geom(scale, C, H, W, PH, PW, S),
       _ptr(rois), _ptr(y))
    _end(lib)
    return y


def backward_nhwc(dy, rois, shape, scale, S, dx=None, assign=False, dev=0, stream=None):
    """dy: cuda [R,PH,PW,C] (fp32, fp16 or bfloat16); shape = (N,H,W,C) of dx, which has dy's type."""
    N, H, W, C = shape
    PH, PW = dy.shape[1], dy.shape[2]
    if dx is None:
        dx = (torch.full(shape, float('nan'), dtype=dy.dtype, device=dy.device) if assign
              else torch.zeros(shape, dtype=dy.dtype, device=dy.device))
    lib = native.library()
    if assign:
        _begin([-1, dy.numel(), -1, -1, -1, -1, -1, -1, -1, -1, dx.numel(), rois.numel()], stream)
        getattr(lib, 'roi_align_backward_nhwc_assign_' + _SUFFIX[dy.dtype][2])(
            ctypes.c_int(dev), ctypes.c_int(dy.numel()), _ptr(dy), *_geom(scale, C, H, W, PH, PW, S),
            ctypes.c_int(N), _ptr(dx), _ptr(rois))
    else:
        _begin([-1, dy.numel(), -1, -1, -1, -1, -1, -1, -1, dx.numel(), rois.numel()], stream)
        getattr(lib, 'roi_align_backward_nhwc_' + _SUFFIX[dy.dtype][1])(
            ctypes.c_int(dev), ctypes.c_int(dy.numel()), _ptr(dy), *_geom(scale, C, H, W, PH, PW, S),
            _ptr(dx), _ptr(rois))
    _end(lib)
    return dx


def set_impl(name):
    native.set_option('roialign_impl', IMPL[name])


def to_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()
